"""Every kernel instantiation the dispatch can choose, forced at small sizes and compared bit for bit
with the CPU oracle: the 2-tile and 4-tile forms of the one-plane prefill kernel (single and grouped
launches), the grouped prefill kernel with one, two and three planes, and the grouped flow kernel on
the 32x32x32 matrix instruction chosen automatically. Precedent: the reference holds its tensor-core
kernel to `to_bits` equality with its dp4a kernel (crates/tritium-cuda/src/cuda/tests.rs:2100-2190)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, bf16_bits_to_f32, f32_to_bf16_bits, rel_err, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def automatic_dispatch(backend):
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)
    backend.set_gemm_tiles(0)
    backend.set_gemm_two_by_two(False)
    backend.set_gemm_rows(0)
    yield
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)
    backend.set_gemm_tiles(0)
    backend.set_gemm_two_by_two(False)
    backend.set_gemm_rows(0)
    backend.set_gemm256_form(-1)
    backend.set_flow_workgroup_waves(0)
    backend.set_stream_min_groups(backend.info.compute_units)


def _set_tiles(backend, tiles):
    """2 = the 64 x 128 form of the one-plane prefill kernel with its four waves side by side (the default
    arrangement), 22 = the same form with the waves two by two, 4 = the 64 x 256 form, 0 = automatic."""
    backend.set_gemm_tiles(2 if tiles == 22 else tiles)
    backend.set_gemm_two_by_two(tiles == 22)


def _planes(rng, n, k, planes):
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    return ws, scs, packed


@pytest.mark.parametrize("tiles", [2, 22, 4])
@pytest.mark.parametrize("m,n,k", [(65, 8, 256), (130, 257, 512), (200, 129, 300), (128, 1040, 2560), (300, 2100, 768)])
def test_one_plane_prefill_kernel_both_tile_counts(backend, oracle, tiles, m, n, k):
    """tk_gemm32_kernel<1,4,false,false,2> (two by two), <1,2,false> and <1,4,false>: ragged tile counts
    (partial workgroups, partial pairs), several row blocks, every output type."""
    print("case gemm-tiles", tiles, m, n, k, flush=True)
    _set_tiles(backend, tiles)
    rng = np.random.default_rng(tiles * 1000 + m + n + k)
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[m // 2] = 0.0
    dact = backend.to_device(act, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    dout = backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    assert same_bits(dout.to_host(), want)
    dob = backend.empty(m * n, "bf16")
    backend.linear_a8(layer, dact, m, dob)
    assert (dob.to_host() == f32_to_bf16_bits(want).reshape(-1)).all()
    # raw accumulators (the int32 the CPU's integer kernel holds before its two multiplies)
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
    backend.linear_i8(layer, dq, None, m, dacc)
    assert (dacc.to_host().reshape(m, n) == oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k)).all()
    # the float contract through the same instantiation
    mf = min(m, 40)
    dof = backend.empty(mf * n, "f32")
    backend.linear_float(layer, dact, mf, dof)
    got = dof.to_host().reshape(mf, n)
    rc, wantf = oracle.cpu_mpgemm(packed[0], FMT_TQ2_0, act[:mf], scs[0], mf, n, k)
    assert rc == 0 and accepts(got, wantf, rel=1e-4, floor=1.0).all()
    for a in (dact, dout, dob, dq, dacc, dof):
        a.free()
    layer.free()


@pytest.mark.parametrize("m,n,k", [(65, 8, 256), (130, 264, 512), (129, 136, 300), (128, 1040, 2560), (300, 2104, 768),
                                   (257, 4104, 256), (640, 520, 1280)])
def test_prefill_kernel_128_rows(backend, oracle, m, n, k):
    """tk_gemm128_kernel forced at small sizes: partial row blocks and column blocks, odd and even half-block
    counts, one to several workgroups per XCD; f32 and bf16 outputs from float rows (with an all-zero token and
    two tokens that hold NaN / Inf and take the reference-order path) and from int8 rows; against the 64-row
    kernels and the CPU oracle, bit for bit. Shapes it does not take fall back to the 64-row kernels."""
    print("case gemm-128", m, n, k, flush=True)
    rng = np.random.default_rng(128000 + m + n + k)
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[m // 2] = 0.0
    act[1, k // 3] = np.nan
    act[m - 1, 0] = np.inf
    dact = backend.to_device(act, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    nan = np.isnan(want)
    got = {}
    for rows in (128, 64):
        backend.set_gemm_rows(rows)
        dout = backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, dout)
        got[rows] = dout.to_host().reshape(m, n)
        assert (np.isnan(got[rows]) == nan).all()
        assert same_bits(got[rows][~nan], want[~nan])
        dob = backend.empty(m * n, "bf16")
        backend.linear_a8(layer, dact, m, dob)
        gb = dob.to_host().reshape(m, n)
        assert (gb[~nan] == f32_to_bf16_bits(want)[~nan]).all()
        dout.free()
        dob.free()
    # int8 rows in, with and without per-token scales
    backend.set_gemm_rows(128)
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    asc = rng.uniform(0.01, 0.2, m).astype(np.float32)
    dq, dsc, do = backend.to_device(q, "i8"), backend.to_device(asc, "f32"), backend.empty(m * n, "f32")
    acc = oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k).astype(np.float32)
    backend.linear_i8(layer, dq, dsc, m, do)
    assert same_bits(do.to_host().reshape(m, n), (acc * scs[0][None, :]) * asc[:, None])
    backend.linear_i8(layer, dq, None, m, do)
    assert same_bits(do.to_host().reshape(m, n), acc * scs[0][None, :])
    for a in (dact, dq, dsc, do):
        a.free()
    layer.free()


@pytest.mark.parametrize("form", [0, 1, 2])
@pytest.mark.parametrize("m,n,k", [(65, 8, 256), (257, 232, 512), (300, 456, 300), (256, 1040, 2560), (520, 2104, 768),
                                   (1030, 4104, 256), (640, 520, 1280), (700, 240, 4096)])
def test_prefill_kernel_256_rows(backend, oracle, m, n, k, form):
    """tk_gemm256_kernel (the weight tile expanded to int8 once per workgroup, in LDS) forced at small sizes, in its three
    forms (four waves of 64 rows, eight waves of 32, and column blocks split over two workgroups): partial row blocks and column blocks (224 outputs each), one and
    several K blocks (odd and even counts: both LDS buffers end a launch), a ragged K, one to several workgroups per
    XCD; f32 and bf16 outputs from float rows (with an all-zero token and two tokens that hold NaN / Inf and take
    the reference-order path) and from int8 rows; against the CPU oracle, bit for bit."""
    print("case gemm-256", m, n, k, form, flush=True)
    rng = np.random.default_rng(256000 + m + n + k)
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[m // 2] = 0.0
    act[1, k // 3] = np.nan
    act[m - 1, 0] = np.inf
    dact = backend.to_device(act, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    nan = np.isnan(want)
    backend.set_gemm_rows(256)
    backend.set_gemm256_form(form)
    dout = backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    assert backend.last_kernel() == "gemm256"
    got = dout.to_host().reshape(m, n)
    assert (np.isnan(got) == nan).all()
    assert same_bits(got[~nan], want[~nan])
    dob = backend.empty(m * n, "bf16")
    backend.linear_a8(layer, dact, m, dob)
    gb = dob.to_host().reshape(m, n)
    assert (gb[~nan] == f32_to_bf16_bits(want)[~nan]).all()
    # int8 rows in, with and without per-token scales
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    asc = rng.uniform(0.01, 0.2, m).astype(np.float32)
    dq, dsc, do = backend.to_device(q, "i8"), backend.to_device(asc, "f32"), backend.empty(m * n, "f32")
    acc = oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k).astype(np.float32)
    backend.linear_i8(layer, dq, dsc, m, do)
    assert backend.last_kernel() == "gemm256"
    assert same_bits(do.to_host().reshape(m, n), (acc * scs[0][None, :]) * asc[:, None])
    backend.linear_i8(layer, dq, None, m, do)
    assert same_bits(do.to_host().reshape(m, n), acc * scs[0][None, :])
    for a in (dact, dout, dob, dq, dsc, do):
        a.free()
    layer.free()


def test_prefill_kernel_128_rows_leaves_other_shapes_alone(backend, oracle):
    """Output rows that are not whole 16-byte pieces, raw accumulators and a fused residual stay with the
    64-row kernels even when 128 rows are asked for."""
    backend.set_gemm_rows(128)
    rng = np.random.default_rng(77)
    m, n, k = 130, 257, 512
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    dact, dout = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    backend.linear_a8(layer, dact, m, dout)
    assert same_bits(dout.to_host(), want)
    q = rng.integers(-128, 128, (m, k)).astype(np.int8)
    dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
    backend.linear_i8(layer, dq, None, m, dacc)
    assert (dacc.to_host().reshape(m, n) == oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k)).all()
    with pytest.raises(T.InvalidInput):
        backend.set_gemm_rows(96)
    for a in (dact, dout, dq, dacc):
        a.free()
    layer.free()


@pytest.mark.parametrize("planes,tiles", [(1, 2), (1, 22), (1, 4), (2, 0), (3, 0)])
def test_grouped_prefill_kernel_every_plane_count(backend, oracle, planes, tiles):
    """A grouped decode launch whose operand rows exceed LDS runs the prefill kernel from a problem
    table: tk_gemm32_kernel<1,2,true>, <1,4,true>, <2,2,true>, <3,2,true>. Members of different widths
    (ragged tile counts), two sharing an activation; one member short enough for the flow kernel's
    share of the group. Bits equal the single launches and the CPU composition."""
    print("case grouped-prefill", planes, tiles, flush=True)
    _set_tiles(backend, tiles)
    rng = np.random.default_rng(planes * 10 + tiles)
    m, k_long, k_short = 40, 4500, 768  # 40 rows x 18 K blocks = 184 KiB of operand rows: beyond LDS
    acts = {"a": rng.standard_normal((m, k_long)).astype(np.float32),
            "b": rng.standard_normal((m, k_long)).astype(np.float32),
            "c": rng.standard_normal((m, k_short)).astype(np.float32)}
    dev = {key: backend.to_device(v, "f32") for key, v in acts.items()}
    members, checks = [], []
    for n, key in ((136, "a"), (200, "c"), (72, "a"), (1050, "b"), (48, "c")):
        k = acts[key].shape[1]
        ws, scs, packed = _planes(rng, n, k, planes)
        layer = backend.linear(packed, scs, n, k)
        out_g, out_s = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
        members.append((layer, dev[key], m, out_g))
        checks.append((layer, dev[key], out_g, out_s, packed, scs, acts[key], n, k))
    grp = backend.group(members, 1, "f32", "f32")
    grp.launch()
    grp.launch()
    for layer, src, out_g, out_s, packed, scs, act, n, k in checks:
        backend.linear_a8(layer, src, m, out_s)
        got = out_g.to_host()
        assert same_bits(got, out_s.to_host())
        assert same_bits(got, oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
    grp.destroy()
    for layer, _, out_g, out_s, *_ in checks:
        out_g.free()
        out_s.free()
        layer.free()
    for d in dev.values():
        d.free()


@pytest.mark.parametrize("mode,m,planes", [(1, 28, 2), (1, 32, 1), (0, 8, 2), (0, 7, 1)])
def test_grouped_flow_kernel_wide_form_chosen_automatically(backend, oracle, mode, m, planes):
    """25..32 operand rows that take at most 64 KiB of LDS: the flow kernel picks the 32x32x32 matrix
    instruction by itself (tk_flow32_kernel<P,1,*,true> from a problem table: the headline's batch 8 is
    8 tokens x 4 digit rows x 2 planes; under the int8 contract, where both forms put the weights first, only
    with two planes). The group is made wide enough for the flow kernel by lowering
    the workgroup threshold, not by forcing a kernel. Forced onto the 16x16x64 form it gives the same
    bits."""
    print("case grouped-flow32", mode, m, planes, flush=True)
    backend.set_stream_min_groups(1)
    rng = np.random.default_rng(mode * 100 + m + planes)
    k = 2048
    act_a = rng.standard_normal((m, k)).astype(np.float32)
    act_b = rng.standard_normal((m, k)).astype(np.float32)
    da, db = backend.to_device(f32_to_bf16_bits(act_a), "bf16"), backend.to_device(f32_to_bf16_bits(act_b), "bf16")
    act_a = bf16_bits_to_f32(f32_to_bf16_bits(act_a)).reshape(m, k)
    act_b = bf16_bits_to_f32(f32_to_bf16_bits(act_b)).reshape(m, k)
    members, checks = [], []
    for n, src, act in ((520, da, act_a), (136, db, act_b), (1029, da, act_a)):
        ws, scs, packed = _planes(rng, n, k, planes)
        layer = backend.linear(packed, scs, n, k)
        out_g, out_s = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
        members.append((layer, src, m, out_g))
        checks.append((layer, src, out_g, out_s, packed, scs, act, n))
    grp = backend.group(members, mode, "bf16", "f32")
    grp.launch()
    grp.launch()
    backend.set_flow_mfma(16)
    grp16 = backend.group([(l, s, m, o) for (l, s, _, o, *_r) in checks], mode, "bf16", "f32")
    for layer, src, out_g, out_s, packed, scs, act, n in checks:
        got = out_g.to_host()
        if mode == 1:
            assert same_bits(got, oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
        else:
            want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
            assert rel_err(got.reshape(m, n), want) <= 1e-3
            assert accepts(got.reshape(m, n), want, rel=1e-4, floor=1.0).all()
    grp16.launch()
    for layer, src, out_g, out_s, *_ in checks:
        assert same_bits(out_g.to_host(), out_s.to_host())  # out_s: the 16x16x64 form's result
    grp.destroy()
    grp16.destroy()
    for layer, _, out_g, out_s, *_ in checks:
        out_g.free()
        out_s.free()
        layer.free()
    da.free()
    db.free()


@pytest.mark.parametrize("mode,m,planes,k", [(1, 22, 1, 2560), (1, 24, 2, 2560), (0, 6, 1, 2560), (1, 17, 1, 3328), (1, 28, 1, 2048), (0, 7, 2, 2048)])
def test_two_row_tiles_in_eight_wave_workgroups(backend, oracle, mode, m, planes, k):
    """17..32 operand rows whose copy in LDS takes between a third of the 160 KiB and 64 KiB: the flow kernels
    run them in eight-wave workgroups (both matrix-instruction forms), single launches and groups. Bits of the
    CPU under the int8 contract, its bounds under the float contract, and the same bits with the run length and
    the ring forced to other values."""
    print("case eight-wave rt2", mode, m, planes, k, flush=True)
    backend.set_stream_min_groups(1)
    rng = np.random.default_rng(mode * 1000 + m * 10 + planes + k)
    n = 1029
    act = rng.standard_normal((m, k)).astype(np.float32)
    dact = backend.to_device(f32_to_bf16_bits(act), "bf16")
    act = bf16_bits_to_f32(f32_to_bf16_bits(act)).reshape(m, k)
    ws, scs, packed = _planes(rng, n, k, planes)
    layer = backend.linear(packed, scs, n, k)
    out, out2 = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
    call = backend.linear_a8 if mode == 1 else backend.linear_float
    call(layer, dact, m, out)
    assert backend.last_kernel() in ("flow", "flow32"), backend.last_kernel()
    got = out.to_host().copy()
    if mode == 1:
        assert same_bits(got, oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
    else:
        want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
        assert rel_err(got.reshape(m, n), want) <= 1e-3
        assert accepts(got.reshape(m, n), want, rel=1e-4, floor=1.0).all()
    try:
        for run_tiles, ring in ((1, 3), (3, 2), (2, 4)):
            backend.set_flow_run_tiles(run_tiles)
            backend.set_flow_ring(ring)
            call(layer, dact, m, out2)
            assert same_bits(out2.to_host(), got), (run_tiles, ring)
            grp = backend.group([(layer, dact, m, out2), (layer, dact, m, out)], mode, "bf16", "f32")
            grp.launch()
            assert same_bits(out2.to_host(), got) and same_bits(out.to_host(), got), (run_tiles, ring)
            grp.destroy()
    finally:
        backend.set_flow_run_tiles(0)
        backend.set_flow_ring(0)
    for x in (dact, out, out2):
        x.free()
    layer.free()


@pytest.mark.parametrize("m,planes,k,n", [(24, 1, 4096, 1029), (32, 1, 4864, 520), (17, 2, 5120 - 40, 1029), (32, 2, 4096, 300), (32, 1, 2560, 1029),
                                          (20, 3, 4096, 134)])
def test_sixteen_wave_workgroups(backend, oracle, m, planes, k, n):
    """17..32 int8 rows whose copy in LDS takes more than 80 KiB, so that a CU runs one workgroup: with sixteen waves
    (tk_flow_kernel<P,2,*,2,*,false,*> at 1024 threads; both operand orders) the bits of eight waves and of the CPU, single launches,
    groups of members of different widths, a member with a zero-chunk map, a residual. The last two cases have no
    form of 1024 threads (rows within 80 KiB; three planes): the setting must leave them on eight waves."""
    print("case sixteen waves", m, planes, k, n, flush=True)
    backend.set_stream_min_groups(1)
    backend.set_decode_kernel(3)
    rng = np.random.default_rng(m * 1000 + planes * 100 + k + n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[m // 2, 7] = np.inf  # a token that the kernel recomputes in the reference's order
    dact = backend.to_device(act, "f32")
    ws, scs, packed = _planes(rng, n, k, planes)
    ws2 = [w.copy() for w in ws]
    ws2[-1][16:64, :] = 0
    ws2[-1][:, 256:1024] = 0
    packed2 = [T.pack_rows(w, n, k) for w in ws2]
    n3 = 136
    ws3, scs3, packed3 = _planes(rng, n3, k, planes)
    layer = backend.linear(packed, scs, n, k)
    backend.set_zero_skip(2)
    layer2 = backend.linear(packed2, scs, n, k)
    backend.set_zero_skip(0)
    layer3 = backend.linear(packed3, scs3, n3, k)
    res = rng.standard_normal((m, n)).astype(np.float32)
    dres = backend.to_device(res, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    want2 = oracle.cpu_linear_a8_planes(packed2, FMT_TQ2_0, scs, act, m, n, k)
    want3 = oracle.cpu_linear_a8_planes(packed3, FMT_TQ2_0, scs3, act, m, n3, k)
    def like_cpu(got, ref):
        got, ref = got.reshape(-1), np.asarray(ref, np.float32).reshape(-1)
        fin = ~np.isnan(ref)
        return bool((np.isnan(got) == np.isnan(ref)).all()) and same_bits(got[fin], ref[fin])
    outs = {}
    try:
        for waves in (16, 8):
            backend.set_flow_workgroup_waves(waves)
            o1, o2, o3, ores, o16 = (backend.empty(m * n, "f32"), backend.empty(m * n, "f32"), backend.empty(m * n3, "f32"),
                                     backend.empty(m * n, "f32"), backend.empty(m * n, "bf16"))
            backend.linear_a8(layer, dact, m, o1)
            assert backend.last_kernel() == "flow", backend.last_kernel()
            backend.linear_a8(layer, dact, m, o16)
            backend.linear_a8_residual(layer, dact, m, dres, ores)
            single = o1.to_host().copy()
            grp = backend.group([(layer, dact, m, o1), (layer2, dact, m, o2), (layer3, dact, m, o3)], 1, "f32", "f32")
            grp.launch()
            grp.launch()
            outs[waves] = [single] + [x.to_host().copy() for x in (o1, o2, o3, ores, o16)]
            grp.destroy()
            backend.set_flow_operand_order(0)  # activations first: the table forms have 1024 threads too
            grp = backend.group([(layer, dact, m, o1), (layer2, dact, m, o2), (layer3, dact, m, o3)], 1, "f32", "f32")
            grp.launch()
            backend.set_flow_operand_order(1)
            for got, ref in zip((o1, o2, o3), outs[waves][1:4]):
                assert same_bits(got.to_host(), ref)
            grp.destroy()
            for x in (o1, o2, o3, ores, o16):
                x.free()
    finally:
        backend.set_flow_workgroup_waves(0)
        backend.set_flow_operand_order(1)
    for a, b in zip(outs[16], outs[8]):
        assert same_bits(a, b)
    assert like_cpu(outs[16][0], want) and like_cpu(outs[16][1], want)
    assert like_cpu(outs[16][2], want2) and like_cpu(outs[16][3], want3)
    assert like_cpu(outs[16][4], (res + want.reshape(m, n)).astype(np.float32))
    for x in (dact, dres):
        x.free()
    for l in (layer, layer2, layer3):
        l.free()


@pytest.mark.parametrize("m,planes,k", [(5, 1, 4096), (8, 1, 4864), (6, 2, 4096), (8, 1, 2048)])
def test_sixteen_wave_workgroups_float_contract(backend, oracle, m, planes, k):
    """5..8 float tokens (20..32 digit rows) beyond 80 KiB in grouped launches: the activations-first forms that read a
    problem table also exist with 1024 threads. Bits of eight waves, bounds of the CPU; single launches (no such
    form) and rows within 80 KiB (last case) stay on eight waves whatever is asked."""
    print("case sixteen waves float", m, planes, k, flush=True)
    backend.set_stream_min_groups(1)
    backend.set_decode_kernel(3)
    rng = np.random.default_rng(m * 1000 + planes * 100 + k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    dact = backend.to_device(f32_to_bf16_bits(act), "bf16")
    act = bf16_bits_to_f32(f32_to_bf16_bits(act)).reshape(m, k)
    sets = []
    for n in (1029, 136):
        ws, scs, packed = _planes(rng, n, k, planes)
        sets.append((n, scs, packed, backend.linear(packed, scs, n, k)))
    outs = {}
    try:
        for waves in (16, 8):
            backend.set_flow_workgroup_waves(waves)
            o = [backend.empty(m * n, "f32") for n, *_ in sets]
            single = backend.empty(m * sets[0][0], "f32")
            grp = backend.group([(st[3], dact, m, oo) for st, oo in zip(sets, o)], 0, "bf16", "f32")
            grp.launch()
            grp.launch()
            backend.linear_float(sets[0][3], dact, m, single)
            assert backend.last_kernel() in ("flow", "flow32"), backend.last_kernel()
            outs[waves] = [x.to_host().copy() for x in o + [single]]
            grp.destroy()
            for x in o + [single]:
                x.free()
    finally:
        backend.set_flow_workgroup_waves(0)
    for a, b in zip(outs[16], outs[8]):
        assert same_bits(a, b)
    assert same_bits(outs[16][0], outs[16][2])  # grouped and single launch
    for (n, scs, packed, _), got in zip(sets, outs[16]):
        want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
        assert rel_err(got.reshape(m, n), want) <= 1e-3
        assert accepts(got.reshape(m, n), want, rel=1e-4, floor=1.0).all()
    dact.free()
    for st in sets:
        st[3].free()


@pytest.mark.parametrize("m", [1, 3, 4, 9, 16, 20, 40, 64])
@pytest.mark.parametrize("planes,n,mfma", [(1, 1029, 0), (2, 520, 0), (3, 134, 0), (4, 48, 0), (1, 1029, 32), (2, 520, 32), (2, 56, 32)])
def test_both_operand_orders_of_the_decode_kernel(backend, oracle, m, planes, n, mfma):
    """The decode kernel under the int8 contract with weights as the first operand of the matrix instruction (a lane
    finishes four channels of one token: one wide store) and with activations first: the same bits, and the CPU's --
    f32 and bf16 outputs, output rows whose stride does not allow the wide store, a residual, a token holding NaN
    (recomputed in the reference's order), single launches and groups; the 16x16x64 form where the library would pick
    it and the 32x32x32 form forced (one and two planes; an odd tile count, so a pair whose second tile does not exist)."""
    print("case operand order", m, planes, n, mfma, flush=True)
    backend.set_stream_min_groups(1)
    backend.set_decode_kernel(3)  # the flow kernel also for launches that would go elsewhere
    backend.set_flow_mfma(mfma)
    rng = np.random.default_rng(m * 100 + planes * 7 + n)
    k = 1280 - 24
    act = rng.standard_normal((m, k)).astype(np.float32)
    if m >= 3:
        act[m // 2, 5] = np.nan
    dact = backend.to_device(act, "f32")
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85, 0.9)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    res = rng.standard_normal((m, n)).astype(np.float32)
    dres = backend.to_device(res, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    outs = {}
    try:
        for order in (1, 0):
            backend.set_flow_operand_order(order)
            o32, o16, ores = backend.empty(m * n, "f32"), backend.empty(m * n, "bf16"), backend.empty(m * n, "f32")
            backend.linear_a8(layer, dact, m, o32)
            assert backend.last_kernel() == ("flow32" if mfma == 32 and m > 16 else "flow"), backend.last_kernel()
            backend.linear_a8(layer, dact, m, o16)
            backend.linear_a8_residual(layer, dact, m, dres, ores)
            g32 = backend.empty(m * n, "f32")
            grp = backend.group([(layer, dact, m, g32), (layer, dact, m, o32)], 1, "f32", "f32")
            grp.launch()
            outs[order] = [x.to_host().copy() for x in (o32, o16, ores, g32)]
            grp.destroy()
            for x in (o32, o16, ores, g32):
                x.free()
    finally:
        backend.set_flow_operand_order(1)
        backend.set_flow_mfma(0)
    for a, b in zip(outs[0], outs[1]):
        assert same_bits(a, b)
    def like_cpu(got, ref):  # (NaN where the CPU has NaN -- the payload may differ -- and its bits everywhere else)
        got, ref = got.reshape(-1), np.asarray(ref, np.float32).reshape(-1)
        fin = ~np.isnan(ref)
        return bool((np.isnan(got) == np.isnan(ref)).all()) and same_bits(got[fin], ref[fin])
    assert like_cpu(outs[1][0], want) and like_cpu(outs[1][3], want)
    assert like_cpu(outs[1][2], (res + want.reshape(m, n)).astype(np.float32))
    for x in (dact, dres):
        x.free()
    layer.free()


def test_gemm_tiles_knob_rejects_other_values(backend):
    for bad in (1, 3, 8, -2):
        with pytest.raises(T.InvalidInput):
            backend.set_gemm_tiles(bad)


@pytest.mark.parametrize("slices", [2, 3, 5, 0])
@pytest.mark.parametrize("m,n,k,planes,tiles", [(64, 200, 2816, 3, 0), (40, 1040, 4352, 1, 2), (40, 1040, 4352, 1, 22), (40, 1040, 4352, 1, 4),
                                                  (100, 50, 1300, 2, 0), (130, 131, 1024, 1, 0)])
def test_prefill_kernel_k_split(backend, oracle, slices, m, n, k, planes, tiles):
    """Single launches of the prefill kernel with K cut into slices (tk_gemm32_kernel<P,NT,false,true>): int32
    partial sums meet in a workspace and the last workgroup to arrive finishes the tile. Bits equal the
    unsplit kernel's and the CPU composition's; a second call reuses the arrival counters (they must be
    back at zero); ragged slice counts (11, 17, 6, 4 K blocks over 2, 3, 5 slices) included."""
    print("case k-split", slices, m, n, k, planes, tiles, flush=True)
    _set_tiles(backend, tiles)
    rng = np.random.default_rng(slices * 1000 + m + n + k)
    ws, scs, packed = _planes(rng, n, k, planes)
    layer = backend.linear(packed, scs, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[1, 3] = np.nan
    dact = backend.to_device(act, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(m, n)
    fin = ~np.isnan(want)
    backend.set_gemm_ksplit(1)
    d0 = backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, d0)
    backend.set_gemm_ksplit(slices)
    try:
        for dtype in ("f32", "bf16"):
            d1 = backend.empty(m * n, dtype)
            for _ in range(2):
                backend.linear_a8(layer, dact, m, d1)
                got = d1.to_host().reshape(m, n)
                if dtype == "f32":
                    assert same_bits(got[fin], want[fin]) and same_bits(got[fin], d0.to_host().reshape(m, n)[fin])
                    assert (np.isnan(got) == ~fin).all()
                else:
                    assert (got[fin] == f32_to_bf16_bits(want).reshape(m, n)[fin]).all()
            d1.free()
        if planes == 1:  # raw accumulators
            q = rng.integers(-128, 128, (m, k)).astype(np.int8)
            dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
            backend.linear_i8(layer, dq, None, m, dacc)
            assert (dacc.to_host().reshape(m, n) == oracle.int8_accumulators(packed[0], FMT_TQ2_0, q, m, n, k)).all()
            dq.free()
            dacc.free()
        # the float contract through the same split
        mf = min(m, 30)
        df = backend.empty(mf * n, "f32")
        backend.linear_float(layer, dact, mf, df)
        wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act[:mf], mf, n, k)
        finf = ~np.isnan(wantf)
        assert accepts(df.to_host().reshape(mf, n)[finf], wantf[finf], rel=1e-4, floor=1.0).all()
        df.free()
    finally:
        backend.set_gemm_ksplit(0)
    for a in (dact, d0):
        a.free()
    layer.free()


@pytest.mark.parametrize("mode", [1, 0])
@pytest.mark.parametrize("k,m,copies", [(256, 1, 40), (2048, 4, 10), (2560, 2, 20), (6912, 3, 12), (17408, 1, 3), (6912, 40, 1),
                                          (2000, 2, 20)])
def test_activation_prep_forms_agree(backend, oracle, mode, k, m, copies):
    """The quantization / digit-split launch has three forms: a wave per token, a workgroup per token (both in
    a straight-line variant for rows of whole K blocks, up to 8 pieces held per thread), and the general
    workgroup-per-token kernels. Forced either way through the knob, a grouped launch of `copies` members must
    give the same bits, and the int8 contract the oracle's (rows with NaN, Inf, all zeros and a single
    non-zero element included; K=2000 is not whole blocks: the general kernels)."""
    print("case prep-forms", mode, k, m, copies, flush=True)
    if mode == 0 and m * 4 > 64:
        pytest.skip("float groups take at most 16 tokens")
    rng = np.random.default_rng(k + m * 7 + copies + mode)
    n = 48
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    acts = []
    for c in range(copies):
        a = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-3, 3)).astype(np.float32)
        if c == 1:
            a[0] = 0.0
        if c == 2:
            a[0] = 0.0
            a[0, k // 2] = -3.25
        if c == 3:
            a[m - 1, 5] = np.nan
        if c == 4:
            a[0, k - 1] = np.inf
        acts.append(a)
    results = []
    for team_rows in (0, 1 << 20):
        backend.set_prep_team_rows(team_rows)
        for dt in ("f32", "bf16"):
            host = [f32_to_bf16_bits(a) if dt == "bf16" else a for a in acts]
            seen = [bf16_bits_to_f32(h).reshape(m, k) if dt == "bf16" else h for h in host]
            dev = [backend.to_device(h, dt) for h in host]
            outs = [backend.empty(m * n, "f32") for _ in range(copies)]
            grp = backend.group([(layer, dev[c], m, outs[c]) for c in range(copies)], mode, dt, "f32")
            grp.launch()
            got = [o.to_host().reshape(m, n) for o in outs]
            results.append(got)
            if mode == 1:
                for c in range(copies):
                    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, seen[c], m, n, k).reshape(m, n)
                    fin = ~np.isnan(want)
                    assert (np.isnan(got[c]) == ~fin).all() and same_bits(got[c][fin], want[fin])
            else:
                for c in range(copies):
                    want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, seen[c], m, n, k).reshape(m, n)
                    fin = ~np.isnan(want)
                    assert (np.isnan(got[c]) == ~fin).all() and accepts(got[c][fin], want[fin], rel=1e-4, floor=1.0).all()
            grp.destroy()
            for x in dev + outs:
                x.free()
    backend.set_prep_team_rows(384)
    for dt_i in range(2):  # same element type, the two settings
        for c in range(copies):
            a, b = results[dt_i][c], results[2 + dt_i][c]
            fin = ~np.isnan(a)
            assert (np.isnan(b) == ~fin).all() and same_bits(a[fin], b[fin])
    layer.free()


@pytest.mark.parametrize("m", [17, 20, 32, 64])
def test_narrow_groups_of_several_row_tiles_take_the_prefill_kernel(backend, oracle, m):
    """q,k,v and gate,up of a decode step of 17..64 tokens are narrow groups (a few hundred tiles) whose rows fit LDS;
    left to the automatic dispatch they run through the grouped prefill kernel (the K-split kernel below 20 rows for the
    small group). Whatever is picked: the CPU oracle's bits, with and without an RMSNorm in front."""
    print("case narrow-group", m, flush=True)
    rng = np.random.default_rng(900 + m)
    h, f, kv = 512, 1536, 128
    x = (rng.standard_normal((m, h)) * 2).astype(np.float32)
    x[m // 2] = 0.0
    dx = backend.to_device(x, "f32")
    nw = rng.uniform(0.5, 1.5, h).astype(np.float32)
    dw = backend.to_device(nw, "f32")
    y = np.stack([oracle.rmsnorm(x[r], nw, 1e-5) for r in range(m)])
    for names in ((h, kv, kv), (f, f)):
        for normed in (True, False):
            members, keep = [], []
            for n in names:
                w, sc = ternary(rng, n, h, 0.4), scales(rng, n)
                packed = T.pack_rows(w, n, h)
                layer = backend.linear([packed], [sc], n, h)
                out = backend.empty(m * n, "f32")
                members.append((layer, dx, m, out))
                keep.append((layer, out, packed, sc, n))
            grp = backend.group(members, 1, "f32", "f32", norms=[(dw, 1e-5, False)] * len(names) if normed else None)
            grp.launch()
            grp.launch()
            for layer, out, packed, sc, n in keep:
                want = oracle.cpu_linear_a8_planes([packed], FMT_TQ2_0, [sc], y if normed else x, m, n, h)
                assert same_bits(out.to_host(), want), (m, n, normed)
            grp.destroy()
            for layer, out, *_ in keep:
                out.free()
                layer.free()
    dx.free()
    dw.free()
