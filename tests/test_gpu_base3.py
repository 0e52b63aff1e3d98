"""Base-3 weight stream: the decode kernel that reads TQ1_0-coded bytes (five trits each, 52 bytes per
256 trits) and decodes them in the kernel, as the reference's base-3 GEMV does per element
(crates/tritium-cuda/kernels/tq2_0_add.cu:744-774; byte code: crates/tritium-format/src/tq1.rs:18-30).
The integers it accumulates are those of the 2-bit kernels, so every output must carry the bits of the
2-bit path and of the CPU oracle: int8 contract bit-exact, float contract bit-equal to the 2-bit kernel
and within the reference's tolerance of the oracle's fold."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, bf16_bits_to_f32, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def flow_for_everything(backend):
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)
    backend.set_stream_min_groups(1)  # the flow kernel also for small launches
    yield
    backend.set_stream_min_groups(backend.info.compute_units)
    backend.set_base3_stream(0)
    backend.set_flow_run_tiles(0)


def test_upload_modes(backend):
    rng = np.random.default_rng(0)
    n, k = 50, 700
    w = ternary(rng, n, k)
    shape = T.GemmShape(0, n, k)
    p2, p1 = T.pack_rows(w, n, k), T.pack_rows(w, n, k, T.TernaryFormat.Tq1_0)
    chunks = 4 * 3
    for mode, want2, want1 in ((0, 0, 0), (1, 0, chunks * 832), (2, chunks * 832, chunks * 832)):
        backend.set_base3_stream(mode)
        b2 = backend.upload_weights(p2, shape, T.TernaryFormat.Tq2_0)
        b1 = backend.upload_weights(p1, shape, T.TernaryFormat.Tq1_0)
        assert (b2.base3_bytes(), b1.base3_bytes()) == (want2, want1)
        assert (b1.download_trits().reshape(n, k) == w).all() and (b2.download_trits().reshape(n, k) == w).all()
        b1.free()
        b2.free()
    with pytest.raises(T.InvalidInput):
        backend.set_base3_stream(3)


@pytest.mark.parametrize("m", [1, 2, 5, 8, 16, 17, 32])
@pytest.mark.parametrize("planes", [1, 2, 3])
@pytest.mark.parametrize("fmt", ["tq1", "tq2"])
def test_bits_equal_the_two_bit_path_and_the_oracle(backend, oracle, m, planes, fmt):
    print("case base3", m, planes, fmt, flush=True)
    rng = np.random.default_rng(m * 100 + planes * 10 + (fmt == "tq1"))
    n, k = 16 * 37 + 5, 256 * 7 - 13  # a ragged last tile and a ragged last K block
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    tfmt, ofmt = (T.TernaryFormat.Tq1_0, FMT_TQ1_0) if fmt == "tq1" else (T.TernaryFormat.Tq2_0, FMT_TQ2_0)
    packed = [T.pack_rows(w, n, k, tfmt) for w in ws]
    backend.set_base3_stream(2)
    native = backend.linear(packed, scs, n, k, tfmt)
    assert all(p.base3_bytes() == 38 * 7 * 832 for p in native.planes)
    backend.set_base3_stream(0)
    plain = backend.linear(packed, scs, n, k, tfmt)
    assert not any(p.base3_bytes() for p in plain.planes)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[0, :7] = [0.0, 1e-3, -1e-3, 3.5, -3.5, 1e3, -1e3]
    bits = f32_to_bf16_bits(act)
    actb = bf16_bits_to_f32(bits).reshape(m, k)
    dact = backend.to_device(bits, "bf16")
    o1, o2 = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    for run_tiles in (0, 1, 3):
        backend.set_flow_run_tiles(run_tiles)
        backend.linear_a8(native, dact, m, o1)
        backend.linear_a8(plain, dact, m, o2)
        want = oracle.cpu_linear_a8_planes(packed, ofmt, scs, actb, m, n, k)
        assert same_bits(o1.to_host(), o2.to_host()) and same_bits(o1.to_host(), want)
    backend.set_flow_run_tiles(0)
    if m <= 8:  # float contract: four digit rows per token, 32 operand rows at most
        backend.linear_float(native, dact, m, o1)
        backend.linear_float(plain, dact, m, o2)
        wantf = oracle.cpu_mpgemm_planes(packed, ofmt, scs, actb, m, n, k)
        assert same_bits(o1.to_host(), o2.to_host())
        assert accepts(o1.to_host().reshape(m, n), wantf, rel=1e-4, floor=1.0).all()
    # grouped: two members on the base-3 copy; then a group that mixes in a member without one (2-bit kernel)
    g1, g2 = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    grp = backend.group([(native, dact, m, g1), (native, dact, m, g2)], 1, "bf16", "f32")
    grp.launch()
    grp.launch()
    assert same_bits(g1.to_host(), want) and same_bits(g2.to_host(), want)
    grp.destroy()
    g1.copy_from(np.zeros(m * n, np.float32))
    grp = backend.group([(native, dact, m, g1), (plain, dact, m, g2)], 1, "bf16", "f32")
    grp.launch()
    assert same_bits(g1.to_host(), want) and same_bits(g2.to_host(), want)
    grp.destroy()
    for a in (dact, o1, o2, g1, g2):
        a.free()
    native.free()
    plain.free()


def test_non_finite_tokens_take_the_reference_order_path(backend, oracle):
    """A token holding NaN or Inf leaves the kernel through the exact fallback, which reads the 2-bit copy."""
    rng = np.random.default_rng(5)
    n, k, m = 200, 1000, 3
    w, sc = ternary(rng, n, k), scales(rng, n)
    packed = T.pack_rows(w, n, k, T.TernaryFormat.Tq1_0)
    backend.set_base3_stream(1)
    layer = backend.linear([packed], [sc], n, k, T.TernaryFormat.Tq1_0)
    assert layer.planes[0].base3_bytes()
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[1, 17] = np.inf
    act[2, 400] = np.nan
    dact, out = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, out)
    rc, want = oracle.cpu_mpgemm(packed, FMT_TQ1_0, act, sc, m, n, k)
    got = out.to_host().reshape(m, n)
    want = want.reshape(m, n)
    fin = ~np.isnan(want)
    assert rc == 0 and (np.isnan(got) == ~fin).all() and np.isnan(got[2]).any() and not np.isnan(got[2]).all()
    assert same_bits(got[1:][fin[1:]], want[1:][fin[1:]]) and accepts(got[0], want[0]).all()
    backend.linear_a8(layer, dact, m, out)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ1_0, act, sc, m, n, k)
    got, want = out.to_host().reshape(m, n), want.reshape(m, n)
    fin = ~np.isnan(want)
    assert rc == 0 and (np.isnan(got) == ~fin).all() and same_bits(got[fin], want[fin])
    dact.free()
    out.free()
    layer.free()


def test_full_size_layer(backend, oracle):
    """K=2560 N=6912 (ten K blocks: the ring of four pads to twelve positions), one plane, TQ1_0 upload,
    batch 1 f32 and batch 4 bf16 through a group of four copies: every output against the oracle."""
    rng = np.random.default_rng(9)
    n, k = 6912, 2560
    w, sc = ternary(rng, n, k), scales(rng, n)
    packed = T.pack_rows(w, n, k, T.TernaryFormat.Tq1_0)
    backend.set_base3_stream(1)
    backend.set_stream_min_groups(backend.info.compute_units)
    layer = backend.linear([packed], [sc], n, k, T.TernaryFormat.Tq1_0)
    act = rng.standard_normal((1, k)).astype(np.float32)
    dact, out = backend.to_device(act, "f32"), backend.empty(n, "f32")
    backend.linear_a8(layer, dact, 1, out)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ1_0, act, sc, 1, n, k)
    assert rc == 0 and same_bits(out.to_host(), want)
    m = 4
    members, outs, acts = [], [], []
    for c in range(4):
        bits = f32_to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
        d, o = backend.to_device(bits, "bf16"), backend.empty(m * n, "f32")
        acts.append((bf16_bits_to_f32(bits).reshape(m, k), d))
        outs.append(o)
        members.append((layer, d, m, o))
    grp = backend.group(members, 1, "bf16", "f32")
    grp.launch()
    for c in (0, 3):
        rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ1_0, acts[c][0], sc, m, n, k)
        assert rc == 0 and same_bits(outs[c].to_host(), want)
    grp.destroy()
    for (_, d), o in zip(acts, outs):
        d.free()
        o.free()
    dact.free()
    out.free()
    layer.free()
