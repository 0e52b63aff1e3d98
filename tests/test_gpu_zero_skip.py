"""Zero-chunk skip: planes with block structure (whole 16-row x 256-trit chunks of zero trits) carry a
map and the flow kernel fetches such chunks from a resident zero chunk. Bits must be identical with and
without the map (the reference's contract for its bitmap kernels: a NULL bitmap is the dense behaviour,
crates/tritium-cuda/kernels/tq2_0_add.cu:327-330), and equal to the CPU oracle's. The threshold is the
reference's 0.5% (crates/tritium-cuda/src/cuda/mod.rs:386)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, f32_to_bf16_bits, bf16_bits_to_f32, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def flow_for_everything(backend):
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)
    backend.set_stream_min_groups(1)  # the flow kernel also for small launches
    yield
    backend.set_stream_min_groups(backend.info.compute_units)
    backend.set_zero_skip(0)
    backend.set_flow_run_tiles(0)


def structured(rng, n, k, p_zero_chunk, p0=0.6):
    """i.i.d. trits with whole chunks (16 rows x 256 trits) zeroed with probability p_zero_chunk."""
    w = ternary(rng, n, k, p0)
    nt, nb = (n + 15) // 16, (k + 255) // 256
    z = rng.random((nt, nb)) < p_zero_chunk
    for t in range(nt):
        for b in range(nb):
            if z[t, b]:
                w[t * 16:(t + 1) * 16, b * 256:(b + 1) * 256] = 0
    return w, int(z.sum())


def test_upload_counts_zero_chunks_and_applies_the_threshold(backend, oracle):
    rng = np.random.default_rng(1)
    n, k = 16 * 40 + 5, 256 * 9 - 30
    w, nz = structured(rng, n, k, 0.3)
    buf = backend.upload_weights(T.pack_rows(w, n, k), T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    zero, total, kept = buf.zero_chunks()
    assert total == 41 * 9 and zero >= nz and kept  # (an i.i.d. chunk is never zero by chance: equality in practice)
    assert zero == nz
    # the per-row bitmaps of the reference agree: a chunk is zero iff its 16 row-blocks are
    bm = oracle.compute_zero_bitmaps(oracle.pack_matrix(w, n, k, FMT_TQ2_0), n, k, 9 * 66)[1]
    rows_zero = np.array([[(bm[r] >> b) & 1 for b in range(9)] for r in range(n)], bool)
    chunks = sum(rows_zero[t * 16:(t + 1) * 16, b].all() for t in range(41) for b in range(9))
    assert chunks == zero
    buf.free()
    # below 0.5%: no map; i.i.d. planes have no zero chunk at all
    w2 = ternary(rng, n, k, 0.85)
    w2[:16, :256] = 0  # 1 of 369 chunks = 0.27%
    buf = backend.upload_weights(T.pack_rows(w2, n, k), T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    assert buf.zero_chunks() == (1, 369, False)
    buf.free()
    w2[16:32, 256:512] = 0  # 2 of 369 = 0.54%
    buf = backend.upload_weights(T.pack_rows(w2, n, k), T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    assert buf.zero_chunks() == (2, 369, True)
    buf.free()
    backend.set_zero_skip(1)
    buf = backend.upload_weights(T.pack_rows(w, n, k), T.GemmShape(0, n, k), T.TernaryFormat.Tq2_0)
    assert buf.zero_chunks()[2] is False
    buf.free()


@pytest.mark.parametrize("m", [1, 4, 16, 40])
@pytest.mark.parametrize("planes", [1, 2, 3])
@pytest.mark.parametrize("run_tiles", [0, 1, 3])
def test_bits_identical_with_and_without_the_map(backend, oracle, m, planes, run_tiles):
    print("case zero-skip", m, planes, run_tiles, flush=True)
    backend.set_flow_run_tiles(run_tiles)
    rng = np.random.default_rng(m * 100 + planes * 10 + run_tiles)
    n, k = 16 * 37 + 5, 256 * 7 - 13
    ws = [structured(rng, n, k, pz, p0)[0] for pz, p0 in ((0.1, 0.4), (0.6, 0.7), (0.95, 0.85))[:planes]]
    ws[-1][:, :] = ws[-1]  # (keep as is)
    if planes == 3:
        ws[2][-21:, :] = 0  # the ragged last tile and the one before it entirely zero
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    backend.set_zero_skip(2)
    with_map = backend.linear(packed, scs, n, k)
    assert all(p.zero_chunks()[2] for p in with_map.planes)
    backend.set_zero_skip(1)
    without = backend.linear(packed, scs, n, k)
    assert not any(p.zero_chunks()[2] for p in without.planes)
    act = rng.standard_normal((m, k)).astype(np.float32)
    bits = f32_to_bf16_bits(act)
    actb = bf16_bits_to_f32(bits).reshape(m, k)
    dact = backend.to_device(bits, "bf16")
    o1, o2 = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    backend.linear_a8(with_map, dact, m, o1)
    backend.linear_a8(without, dact, m, o2)
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, actb, m, n, k)
    assert same_bits(o1.to_host(), o2.to_host()) and same_bits(o1.to_host(), want)
    if m <= 16:
        backend.linear_float(with_map, dact, m, o1)
        backend.linear_float(without, dact, m, o2)
        wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, actb, m, n, k)
        assert same_bits(o1.to_host(), o2.to_host())
        assert accepts(o1.to_host().reshape(m, n), wantf, rel=1e-4, floor=1.0).all()
    # a group mixing a mapped and an unmapped member
    g1, g2 = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    grp = backend.group([(with_map, dact, m, g1), (without, dact, m, g2)], 1, "bf16", "f32")
    grp.launch()
    assert same_bits(g1.to_host(), want) and same_bits(g2.to_host(), want)
    grp.destroy()
    for a in (dact, o1, o2, g1, g2):
        a.free()
    with_map.free()
    without.free()


@pytest.mark.parametrize("m", [5, 8, 20, 28, 32, 48, 64])
@pytest.mark.parametrize("planes", [1, 2])
@pytest.mark.parametrize("mfma", [0, 32])
def test_the_32x32x32_form_consults_the_maps_too(backend, oracle, m, planes, mfma):
    """The 32x32x32 form of the flow kernel (automatic at 25..32 operand rows -- with weights as the first operand only
    for two planes --, forced here beyond) with mapped
    planes, single launches and groups: the bits of the unmapped planes and of the CPU. A wave of that form walks a
    pair of tiles, so pairs with one marked chunk, with both and with none all occur."""
    print("case zero-skip 32x32x32", m, planes, mfma, flush=True)
    rng = np.random.default_rng(7000 + m * 100 + planes * 10 + mfma)
    n, k = 16 * 37 + 5, 256 * 7 - 13  # (an odd tile count: the last pair has one tile)
    ws = [structured(rng, n, k, pz, p0)[0] for pz, p0 in ((0.5, 0.4), (0.75, 0.7))[:planes]]
    ws[-1][16:48, :] = 0  # a pair of tiles whose every chunk is marked
    ws[-1][-5:, :256] = 0
    ws[-1][-21:-5, :256] = 0  # ... and the first chunks of the last two tiles
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    backend.set_zero_skip(2)
    with_map = backend.linear(packed, scs, n, k)
    backend.set_zero_skip(1)
    without = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    bits = f32_to_bf16_bits(act)
    actb = bf16_bits_to_f32(bits).reshape(m, k)
    dact = backend.to_device(bits, "bf16")
    o = [backend.empty(m * n, "f32") for _ in range(2)]
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, actb, m, n, k)
    backend.set_flow_mfma(mfma)
    try:
        for weights_first in (0, 1):  # both operand orders of the matrix instruction
            backend.set_flow_operand_order(weights_first)
            backend.linear_a8(with_map, dact, m, o[0])
            took = backend.last_kernel()
            backend.linear_a8(without, dact, m, o[1])
            if mfma == 32 and m > 16 or (24 < m <= 32 and (planes == 2 or not weights_first)):
                assert took == "flow32", (took, m, planes, mfma, weights_first)
            assert same_bits(o[0].to_host(), want) and same_bits(o[1].to_host(), want)
        if m <= 16:
            backend.linear_float(with_map, dact, m, o[0])
            tookf = backend.last_kernel()
            backend.linear_float(without, dact, m, o[1])
            if mfma == 32 or m == 8:
                assert tookf == "flow32", (tookf, m, planes, mfma)
            assert same_bits(o[0].to_host(), o[1].to_host())
            wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, actb, m, n, k)
            assert accepts(o[0].to_host().reshape(m, n), wantf, rel=1e-4, floor=1.0).all()
        # a group of a mapped and an unmapped member through the table forms
        grp = backend.group([(with_map, dact, m, o[0]), (without, dact, m, o[1])], 1, "bf16", "f32")
        grp.launch()
        assert same_bits(o[0].to_host(), want) and same_bits(o[1].to_host(), want)
        grp.destroy()
    finally:
        backend.set_flow_mfma(0)
        backend.set_flow_operand_order(1)
    for a in [dact] + o:
        a.free()
    with_map.free()
    without.free()
