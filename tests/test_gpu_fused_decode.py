"""Single decode calls of one to four tokens run as ONE launch: the decode kernel (the K-split kernel of narrow
launches and the flow kernel of wide ones) quantizes (W1.58A8) or digit-splits (float contract) the tokens itself.
The launch must carry the bits of the two-launch form (same arithmetic, statement for statement) -- and under the
int8 contract the CPU oracle's -- for every plane count, element type, ring size and runs-per-wave form, for rows that are all zero, hold one element, NaN, Inf or a range the digit
grid does not carry (those take the exact fallback inside the kernel), and with a residual. Shapes the form does
not take (K beyond 8192 or not whole blocks, more than four tokens, unaligned rows, RMSNorm in front) must fall
through to the two launches. Reference behaviour for the special rows: crates/tritium-spec/src/lib.rs:351-378,
crates/tritium-core/src/reference.rs:42-51."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, bf16_bits_to_f32, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu

KSPLIT, FLOW = 1, 3


@pytest.fixture(autouse=True, params=[KSPLIT, FLOW], ids=["ksplit", "flow"])
def kernel(request, backend):
    backend.set_decode_kernel(request.param)
    backend.set_fuse_tokens(4)
    yield request.param
    backend.set_decode_kernel(0)
    backend.set_fuse_tokens(-1)
    backend.set_flow_ring(0)


def _takes_one_launch(kernel, float_contract, m, k, planes):
    """The library's rule: whole K blocks up to 8192, and the operand rows (256 bytes per K block and row; four rows
    per token under the float contract) within 62 KiB of LDS for the flow kernel, within the 48 KiB that the
    K-split kernel stages in one pass."""
    nb, rows = k // 256, (4 * m if float_contract else m)
    if k % 256 or nb * 16 > 512 or m > 4:
        return False
    if kernel == FLOW:
        return nb * 256 * rows + 2048 <= 65536
    return nb * 256 * rows <= 48 * 1024


def _planes(rng, n, k, planes):
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    return ws, scs, [T.pack_rows(w, n, k) for w in ws]


def _tokens(rng, m, k, special):
    a = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-2, 3)).astype(np.float32)
    if special == "zero":
        a[0] = 0.0
    elif special == "single":
        a[m - 1] = 0.0
        a[m - 1, k // 3] = -3.25
    elif special == "nan":
        a[0, 5] = np.nan
    elif special == "inf":
        a[m - 1, k - 1] = -np.inf
    elif special == "narrow":  # one element 2^30 times the rest: the digit grid does not carry the small ones
        a[0] = (rng.standard_normal(k) * 1e-3).astype(np.float32)
        a[0, 7] = np.float32(2.0 ** 20)
    return a


def _same(a, b):
    fin = ~np.isnan(a)
    return (np.isnan(b) == ~fin).all() and same_bits(a[fin], b[fin])


@pytest.mark.parametrize("special", ["plain", "zero", "single", "nan", "inf", "narrow"])
@pytest.mark.parametrize("m,n,k,planes", [(1, 48, 256, 1), (1, 6912, 2560, 1), (2, 200, 2048, 2), (3, 130, 5120, 3),
                                            (4, 64, 3840, 1), (4, 96, 1024, 2), (1, 40, 8192, 2), (2, 33, 6912, 1)])
def test_one_launch_equals_two_launches(backend, oracle, kernel, m, n, k, planes, special):
    print("case fused-decode", kernel, m, n, k, planes, special, flush=True)
    rng = np.random.default_rng(m * 1000 + n + k + planes + len(special))
    ws, scs, packed = _planes(rng, n, k, planes)
    layer = backend.linear(packed, scs, n, k)
    act = _tokens(rng, m, k, special)
    for dt in ("f32", "bf16"):
        host = f32_to_bf16_bits(act) if dt == "bf16" else act
        seen = bf16_bits_to_f32(host).reshape(m, k) if dt == "bf16" else act
        dact = backend.to_device(host, dt)
        for odt in ("f32", "bf16"):
            out = backend.empty(m * n, odt)
            for call, name in ((backend.linear_a8, "a8"), (backend.linear_float, "float")):
                got = {}
                for fuse in (4, 0):
                    backend.set_fuse_tokens(fuse)
                    before = backend.fused_calls()
                    call(layer, dact, m, out)
                    got[fuse] = out.to_host().copy()
                    one = fuse and _takes_one_launch(kernel, name == "float", m, k, planes)
                    assert backend.fused_calls() - before == (1 if one else 0), (name, dt, odt, fuse)
                if odt == "bf16":
                    assert (got[4] == got[0]).all() or _same(bf16_bits_to_f32(got[4]), bf16_bits_to_f32(got[0]))
                else:
                    assert _same(got[4], got[0]), (name, dt, odt)
                if odt == "f32" and name == "a8":
                    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, seen, m, n, k)
                    assert _same(want.reshape(-1), got[4].reshape(-1))
                if odt == "f32" and name == "float":
                    want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, seen, m, n, k).reshape(-1)
                    fin = np.isfinite(want)
                    top = max(float(np.abs(want[fin]).max()) if fin.any() else 0.0, 1e-30)
                    assert accepts(got[4].reshape(-1)[fin], want[fin], rel=1e-4, floor=top).all()
            out.free()
        dact.free()
    layer.free()


@pytest.mark.parametrize("ring", [2, 3, 4, 5])
@pytest.mark.parametrize("m,planes", [(1, 1), (2, 1), (1, 2), (3, 3)])
def test_every_ring_size_and_run_count(backend, oracle, kernel, ring, m, planes):
    """The ring of loads (2..5 positions) and one or two runs per wave are separate instantiations of the flow kernel."""
    if kernel != FLOW:
        pytest.skip("the ring belongs to the flow kernel")
    print("case fused-decode ring", ring, m, planes, flush=True)
    rng = np.random.default_rng(ring * 10 + m + planes)
    n, k = 272, 2560
    ws, scs, packed = _planes(rng, n, k, planes)
    layer = backend.linear(packed, scs, n, k)
    backend.set_flow_ring(ring)
    act = _tokens(rng, m, k, "plain")
    dact = backend.to_device(act, "f32")
    out = backend.empty(m * n, "f32")
    before = backend.fused_calls()
    backend.linear_a8(layer, dact, m, out)
    assert backend.fused_calls() == before + 1
    assert same_bits(out.to_host(), oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
    backend.linear_float(layer, dact, m, out)
    got = out.to_host().copy()
    backend.set_fuse_tokens(0)
    backend.linear_float(layer, dact, m, out)
    assert same_bits(got, out.to_host())
    for x in (dact, out):
        x.free()
    layer.free()


def test_residual_rides_along(backend, oracle):
    rng = np.random.default_rng(77)
    m, n, k = 2, 160, 2048
    ws, scs, packed = _planes(rng, n, k, 2)
    layer = backend.linear(packed, scs, n, k)
    act = _tokens(rng, m, k, "plain")
    res = rng.standard_normal((m, n)).astype(np.float32)
    dact, dres, out = backend.to_device(act, "f32"), backend.to_device(res, "f32"), backend.empty(m * n, "f32")
    before = backend.fused_calls()
    backend.linear_a8_residual(layer, dact, m, dres, out)
    assert backend.fused_calls() == before + 1
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(m, n) + res
    assert same_bits(out.to_host().reshape(m, n), want.astype(np.float32))
    for x in (dact, dres, out):
        x.free()
    layer.free()


@pytest.mark.parametrize("m,k,why", [(5, 2048, "tokens"), (1, 8448, "K beyond two pieces per thread"),
                                      (1, 2000, "K not whole blocks"), (4, 4096, "rows beyond 63 KiB of LDS (float contract)")])
def test_other_shapes_take_two_launches(backend, oracle, kernel, m, k, why):
    print("case fused-decode fallthrough", kernel, m, k, why, flush=True)
    rng = np.random.default_rng(m + k)
    n = 80
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = _tokens(rng, m, k, "plain")
    dact, out = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
    before = backend.fused_calls()
    backend.linear_float(layer, dact, m, out)
    assert backend.fused_calls() == before, why
    want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act, m, n, k).reshape(-1)
    assert accepts(out.to_host(), want, rel=1e-4, floor=float(np.abs(want).max())).all()
    backend.linear_a8(layer, dact, m, out)
    assert same_bits(out.to_host(), oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
    for x in (dact, out):
        x.free()
    layer.free()


def test_automatic_dispatch_takes_one_launch_for_one_token(backend, oracle):
    """Left to itself (no kernel forced, the knob on automatic) a one-token call on a layer of configs[0]'s shape is a
    single launch under both contracts; two tokens under the int8 contract only; four under neither."""
    backend.set_decode_kernel(0)
    backend.set_fuse_tokens(-1)
    rng = np.random.default_rng(5)
    n, k = 6912, 2560
    ws, scs, packed = _planes(rng, n, k, 1)
    layer = backend.linear(packed, scs, n, k)
    act = _tokens(rng, 1, k, "plain")
    dact, out = backend.to_device(act, "f32"), backend.empty(n, "f32")
    before = backend.fused_calls()
    backend.linear_a8(layer, dact, 1, out)
    backend.linear_float(layer, dact, 1, out)
    assert backend.fused_calls() == before + 2
    for x in (dact, out):
        x.free()
    for m, expect in ((2, 1), (4, 0)):
        act = _tokens(rng, m, k, "plain")
        dact, out = backend.to_device(act, "f32"), backend.empty(m * n, "f32")
        before = backend.fused_calls()
        backend.linear_a8(layer, dact, m, out)
        assert same_bits(out.to_host(), oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
        backend.linear_float(layer, dact, m, out)
        assert backend.fused_calls() == before + expect, m
        for x in (dact, out):
            x.free()
    layer.free()


@pytest.mark.parametrize("special", ["plain", "zero", "nan", "inf"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("m,normed", [(1, True), (1, False), (2, False), (2, True)])
def test_group_of_single_tokens_is_one_launch(backend, oracle, kernel, m, normed, dtype, special):
    """q,k,v behind the attention norm, o on another tensor, gate,up behind a zero-centred norm, as one group: with one
    token per member the K-split kernel builds every member's rows (norm included) itself. Same bits as the single
    two-launch calls; two tokens behind a norm keep the prep launch."""
    if kernel != KSPLIT:
        pytest.skip("groups take the form in the K-split kernel")
    print("case fused-group", m, normed, dtype, special, flush=True)
    backend.set_decode_kernel(0)
    rng = np.random.default_rng(m * 7 + normed + len(special))
    h, f, kv = 512, 1280, 128
    hid_h, att_h = _tokens(rng, m, h, special), _tokens(rng, m, h, "plain")
    conv = (lambda a: f32_to_bf16_bits(a)) if dtype == "bf16" else (lambda a: a)
    hid, att = backend.to_device(conv(hid_h), dtype), backend.to_device(conv(att_h), dtype)
    w1 = backend.to_device(rng.uniform(0.5, 1.5, h).astype(np.float32), "f32")
    w2 = backend.to_device(rng.uniform(-0.5, 0.5, h).astype(np.float32), "f32")
    n1, n2 = ((w1, 1e-5, False), (w2, 1e-5, True)) if normed else (None, None)
    spec = [("q", h, hid, n1), ("k", kv, hid, n1), ("v", kv, hid, n1), ("o", h, att, None), ("gate", f, hid, n2), ("up", f, hid, n2)]
    members, norms, singles = [], [], []
    for name, n, src, nm in spec:
        layer = backend.linear([T.pack_rows(ternary(rng, n, h, 0.4), n, h)], [scales(rng, n)], n, h)
        members.append((layer, src, m, backend.empty(m * n, "f32")))
        norms.append(nm)
        singles.append(backend.empty(m * n, "f32"))
    backend.set_fuse_tokens(4)
    grp = backend.group(members, 1, dtype, "f32", norms=norms if normed else None)
    before = backend.fused_calls()
    grp.launch()
    grp.launch()
    one = not (normed and m > 1)
    assert backend.fused_calls() - before == (2 if one else 0)
    backend.set_fuse_tokens(0)
    for (layer, src, _, out_g), nm, out_s in zip(members, norms, singles):
        if nm is None:
            backend.linear_a8(layer, src, m, out_s)
        else:
            backend.linear_rmsnorm_a8(layer, src, nm[0], nm[1], m, out_s, zero_centered=nm[2])
        assert _same(out_s.to_host(), out_g.to_host()), (m, normed, dtype, special)
    if not normed:  # the float contract has groups too (no norm there)
        backend.set_fuse_tokens(4)
        fmembers = [(layer, src, m, backend.empty(m * layer.n, "f32")) for (layer, src, _, _) in members]
        fgrp = backend.group(fmembers, 0, dtype, "f32")
        before = backend.fused_calls()
        fgrp.launch()
        assert backend.fused_calls() == before + 1
        backend.set_fuse_tokens(0)
        for (layer, src, _, out_g), out_s in zip(fmembers, singles):
            backend.linear_float(layer, src, m, out_s)
            assert _same(out_s.to_host(), out_g.to_host())
        fgrp.destroy()
        for mem in fmembers:
            mem[3].free()
    grp.destroy()
    for (layer, _, _, out_g), out_s in zip(members, singles):
        out_g.free()
        out_s.free()
        layer.free()
    for a in (hid, att, w1, w2):
        a.free()


@pytest.mark.parametrize("special", ["plain", "zero", "nan", "narrow"])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("planes,normed", [(1, True), (1, False), (2, True), (3, False)])
def test_wide_group_of_single_tokens_is_one_launch_of_the_flow_kernel(backend, oracle, kernel, planes, normed, dtype, special):
    """gate,up of a wide FFN behind a norm, one token: more than two tiles per CU, so the automatic dispatch takes the
    flow kernel, and with one or two planes that kernel builds every member's row (norm included) itself: one launch.
    Same bits as the single two-launch calls, under both contracts; three planes keep the prep launch."""
    if kernel != FLOW:
        pytest.skip("the automatic dispatch is what is tested: once")
    print("case fused-flow-group", planes, normed, dtype, special, flush=True)
    backend.set_decode_kernel(0)
    rng = np.random.default_rng(planes * 11 + normed + len(special))
    h, f = 768, 16 * 257 + 5  # two members of 258 tiles
    hid_h = _tokens(rng, 1, h, special)
    conv = (lambda a: f32_to_bf16_bits(a)) if dtype == "bf16" else (lambda a: a)
    hid = backend.to_device(conv(hid_h), dtype)
    w2 = backend.to_device(rng.uniform(-0.5, 0.5, h).astype(np.float32), "f32")
    nm = (w2, 1e-5, True) if normed else None
    members, singles = [], []
    for _ in range(2):
        ws, scs, packed = _planes(rng, f, h, planes)
        layer = backend.linear(packed, scs, f, h)
        members.append((layer, hid, 1, backend.empty(f, "f32")))
        singles.append(backend.empty(f, "f32"))
    backend.set_fuse_tokens(-1)
    grp = backend.group(members, 1, dtype, "f32", norms=[nm, nm] if normed else None)
    before = backend.fused_calls()
    grp.launch()
    grp.launch()
    # (three planes: the flow kernel has no such form from a table, the K-split kernel would have counted two)
    assert backend.fused_calls() - before == (2 if planes <= 2 else 0)
    backend.set_fuse_tokens(0)
    for (layer, src, _, out_g), out_s in zip(members, singles):
        if nm is None:
            backend.linear_a8(layer, src, 1, out_s)
        else:
            backend.linear_rmsnorm_a8(layer, src, nm[0], nm[1], 1, out_s, zero_centered=nm[2])
        assert _same(out_s.to_host(), out_g.to_host()), (planes, normed, dtype, special)
    if not normed:
        backend.set_fuse_tokens(-1)
        fmembers = [(layer, src, 1, backend.empty(f, "f32")) for (layer, src, _, _) in members]
        fgrp = backend.group(fmembers, 0, dtype, "f32")
        before = backend.fused_calls()
        fgrp.launch()
        assert backend.fused_calls() - before == (1 if planes <= 2 else 0)
        backend.set_fuse_tokens(0)
        for (layer, src, _, out_g), out_s in zip(fmembers, singles):
            backend.linear_float(layer, src, 1, out_s)
            assert _same(out_s.to_host(), out_g.to_host())
        fgrp.destroy()
        for mem in fmembers:
            mem[3].free()
    grp.destroy()
    for (layer, _, _, out_g), out_s in zip(members, singles):
        out_g.free()
        out_s.free()
        layer.free()
    for a in (hid, w2):
        a.free()


def test_group_with_members_of_different_k_and_token_counts(backend, oracle, kernel):
    """One launch for a group whose members differ in K, N, token count and norm: every workgroup sizes its rows, row
    constants and norm scratch from its own member."""
    if kernel != KSPLIT:
        pytest.skip("groups take the form in the K-split kernel")
    backend.set_decode_kernel(0)
    backend.set_fuse_tokens(4)
    rng = np.random.default_rng(21)
    spec = [(1, 80, 512, True), (2, 48, 1280, False), (1, 200, 2560, True), (3, 33, 256, False), (1, 64, 6912, False)]
    members, norms, keep = [], [], []
    for m, n, k, normed in spec:
        w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
        layer = backend.linear([T.pack_rows(w, n, k)], [sc], n, k)
        x = _tokens(rng, m, k, "plain")
        nw = rng.uniform(0.5, 1.5, k).astype(np.float32)
        dx, dw, out = backend.to_device(x, "f32"), backend.to_device(nw, "f32"), backend.empty(m * n, "f32")
        members.append((layer, dx, m, out))
        norms.append((dw, 1e-5, False) if normed else None)
        keep.append((layer, dx, dw, out, x, nw, w, sc, m, n, k, normed))
    grp = backend.group(members, 1, "f32", "f32", norms=norms)
    before = backend.fused_calls()
    grp.launch()
    assert backend.fused_calls() == before + 1
    for layer, dx, dw, out, x, nw, w, sc, m, n, k, normed in keep:
        y = np.stack([oracle.rmsnorm(x[r], nw, 1e-5) for r in range(m)]) if normed else x
        want = oracle.cpu_linear_a8_planes([T.pack_rows(w, n, k)], FMT_TQ2_0, [sc], y, m, n, k)
        assert same_bits(out.to_host(), want), (m, n, k, normed)
    grp.destroy()
    for layer, dx, dw, out, *_ in keep:
        for a in (dx, dw, out):
            a.free()
        layer.free()


@pytest.mark.parametrize("n", [8208, 16384, 20000])
def test_wide_launches_take_several_tiles_per_workgroup(backend, oracle, kernel, n):
    """Beyond two output tiles per CU a workgroup of the K-split form stages its rows once and takes up to four
    consecutive tiles (513 tiles: the last workgroup has one; 1250 tiles: three per workgroup, the last has two).
    Single calls and a group of two members behind a norm, against the oracle's bits."""
    if kernel != KSPLIT:
        pytest.skip("the K-split kernel's form")
    print("case fused-wide", n, flush=True)
    rng = np.random.default_rng(n)
    k = 1024
    w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [sc], n, k)
    for m in (1, 2):
        x = _tokens(rng, m, k, "nan" if m == 2 else "plain")
        dx, out = backend.to_device(x, "f32"), backend.empty(m * n, "f32")
        before = backend.fused_calls()
        backend.linear_a8(layer, dx, m, out)
        assert backend.fused_calls() == before + 1
        assert _same(oracle.cpu_linear_a8_planes([packed], FMT_TQ2_0, [sc], x, m, n, k).reshape(-1), out.to_host())
        backend.linear_float(layer, dx, m, out)
        got = out.to_host().copy()
        backend.set_fuse_tokens(0)
        backend.linear_float(layer, dx, m, out)
        backend.set_fuse_tokens(4)
        assert _same(out.to_host(), got)
        for a in (dx, out):
            a.free()
    x = _tokens(rng, 1, k, "plain")
    nw = rng.uniform(0.5, 1.5, k).astype(np.float32)
    dx, dw = backend.to_device(x, "f32"), backend.to_device(nw, "f32")
    outs = [backend.empty(n, "f32") for _ in range(2)]
    grp = backend.group([(layer, dx, 1, o) for o in outs], 1, "f32", "f32", norms=[(dw, 1e-5, True)] * 2)
    before = backend.fused_calls()
    grp.launch()
    assert backend.fused_calls() == before + (1 if 2 * ((n + 15) // 16) <= 2048 else 0)
    y = oracle.rmsnorm(x[0], nw, 1e-5, True).reshape(1, k)
    want = oracle.cpu_linear_a8_planes([packed], FMT_TQ2_0, [sc], y, 1, n, k).reshape(-1)
    for o in outs:
        assert same_bits(o.to_host(), want)
    grp.destroy()
    for a in [dx, dw] + outs:
        a.free()
    layer.free()


def test_single_call_behind_a_norm_is_one_launch(backend, oracle, kernel):
    """tk_linear_rmsnorm_a8 on one token: norm, quantization and contraction in one launch, the oracle's bits (a row
    with an Inf goes through the exact fallback, which reads the normalized row from LDS)."""
    print("case fused-normed-single", kernel, flush=True)
    rng = np.random.default_rng(11)
    n, k = 6912, 2560
    ws, scs, packed = _planes(rng, n, k, 2)
    layer = backend.linear(packed, scs, n, k)
    w = rng.uniform(0.5, 1.5, k).astype(np.float32)
    dw = backend.to_device(w, "f32")
    for special in ("plain", "inf", "zero"):
        x = _tokens(rng, 1, k, special)
        y = oracle.rmsnorm(x[0], w, 1e-5).reshape(1, k)
        want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, y, 1, n, k).reshape(-1)
        dx, out = backend.to_device(x, "f32"), backend.empty(n, "f32")
        got = {}
        for fuse in (4, 0):
            backend.set_fuse_tokens(fuse)
            before = backend.fused_calls()
            backend.linear_rmsnorm_a8(layer, dx, dw, 1e-5, 1, out)
            assert backend.fused_calls() - before == (1 if fuse else 0)
            got[fuse] = out.to_host().copy()
        assert _same(got[0], got[4]) and _same(want, got[4]), special
        for a in (dx, out):
            a.free()
    dw.free()
    layer.free()


def test_knob_rejects_other_values(backend):
    with pytest.raises(T.BackendError):
        backend.set_fuse_tokens(5)
    with pytest.raises(T.BackendError):
        backend.set_fuse_tokens(-2)
