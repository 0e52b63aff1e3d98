"""BASELINE-size checks: size-independent properties at full shapes plus sampled oracle rows."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import a8_expected, accepts, bf16_bits_to_f32, f32_to_bf16_bits, rel_err, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


def test_config1_full_size(backend, oracle):
    """K=2560, N=6912, 1 plane, f32 N(0,1) activation, batch 1, seed 0: every output against the oracle."""
    rng = np.random.default_rng(0)
    n, k = 6912, 2560
    w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
    act = rng.standard_normal((1, k)).astype(np.float32)
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [sc], n, k)
    dact, dout = backend.to_device(act, "f32"), backend.empty(n, "f32")
    backend.linear_float(layer, dact, 1, dout)
    got = dout.to_host()
    rc, want = oracle.cpu_mpgemm(packed, FMT_TQ2_0, act, sc, 1, n, k)
    assert rc == 0 and rel_err(got, want) <= 1e-3 and accepts(got, want.reshape(-1)).all()
    # all-(+1) plane: every output is scale·Σa (closed form)
    ones = T.pack_rows(np.ones((n, k), np.int8), n, k)
    l1 = backend.linear([ones], [np.ones(n, np.float32)], n, k)
    backend.linear_float(l1, dact, 1, dout)
    s = act.astype(np.float64).sum()
    assert np.abs(dout.to_host() - s).max() <= 1e-5 * max(1, abs(s))
    # W1.58A8 at the same size, bit-exact
    backend.linear_a8(layer, dact, 1, dout)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act, sc, 1, n, k)
    assert same_bits(dout.to_host(), want)


def test_config3_prefill_sampled(backend, oracle):
    """M=2048, K=2560, N=6912: int32 accumulators of sampled tokens against the oracle, and
    linearity q -> -q over the whole output."""
    rng = np.random.default_rng(3)
    m, n, k = 2048, 6912, 2560
    w = ternary(rng, n, k, 0.4)
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [np.ones(n, np.float32)], n, k)
    q = rng.integers(-127, 128, (m, k)).astype(np.int8)
    dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
    backend.linear_i8(layer, dq, None, m, dacc)
    acc = dacc.to_host().reshape(m, n)
    rows = [0, 1, 777, 1023, 1024, 2047]
    want = oracle.int8_accumulators(packed, FMT_TQ2_0, q[rows], len(rows), n, k)
    assert (acc[rows] == want).all()
    dq.copy_from(-q)
    backend.linear_i8(layer, dq, None, m, dacc)
    assert (dacc.to_host().reshape(m, n) == -acc).all()
    # column sums: Σ_m acc[m,n] == (Σ_m q[m,:]) · w[n,:]  (a checksum over every token)
    colsum = q.astype(np.int64).sum(axis=0)
    assert (acc.astype(np.int64).sum(axis=0) == w.astype(np.int64) @ colsum).all()


def _bf16(x):
    bits = f32_to_bf16_bits(x)
    return bits, bf16_bits_to_f32(bits).reshape(x.shape)


@pytest.mark.parametrize("m", [1, 32])
def test_config4_projection_stack_group(backend, oracle, m):
    """configs[3] as the benchmark launches it: 30 layers x (q,k,v,o,gate,up,down), hidden 2560, FFN
    6912, 20/5 heads of 128, one plane, W1.58A8, bf16 in and out, ONE grouped launch of 210 members
    (the layers share one set of weights here; inputs and outputs are per layer). At 32 tokens the
    K=6912 down projections exceed LDS and take the grouped prefill kernel. Every output of the first
    and last layer against the exact composition; sampled tokens of it against the C oracle."""
    h, f, kv, layers_n = 2560, 6912, 640, 30
    shapes = {"q": (h, h), "k": (kv, h), "v": (kv, h), "o": (h, h), "gate": (f, h), "up": (f, h), "down": (h, f)}
    rng = np.random.default_rng(40 + m)
    host = {}
    for name, (n, k) in shapes.items():
        w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
        host[name] = (w, sc, T.pack_rows(w, n, k))
    lin = {name: backend.linear([host[name][2]], [host[name][1]], *shapes[name]) for name in shapes}
    srcs, members, outs = [], [], []
    for li in range(layers_n):
        acts = {key: _bf16(rng.standard_normal((m, kk)).astype(np.float32)) for key, kk in (("hid", h), ("att", h), ("mid", f))}
        dev = {key: backend.to_device(bits, "bf16") for key, (bits, _) in acts.items()}
        srcs.append((acts, dev))
        for name, key in (("q", "hid"), ("k", "hid"), ("v", "hid"), ("o", "att"), ("gate", "hid"), ("up", "hid"), ("down", "mid")):
            o = backend.empty(m * shapes[name][0], "bf16")
            outs.append((li, name, key, o))
            members.append((lin[name], dev[key], m, o))
    grp = backend.group(members, 1, "bf16", "bf16")
    grp.launch()
    grp.launch()
    tok = sorted({0, m // 2, m - 1})
    for li, name, key, o in outs:
        if li not in (0, layers_n - 1):
            continue
        print("case config4-stack", m, li, name, flush=True)
        n, k = shapes[name]
        w, sc, packed = host[name]
        act = srcs[li][0][key][1]
        got = o.to_host().reshape(m, n)
        want = a8_expected(oracle, [w], [sc], act)
        assert (got == f32_to_bf16_bits(want).reshape(m, n)).all()
        rc, ref = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act[tok], sc, len(tok), n, k)
        assert rc == 0 and same_bits(want[tok], ref)
    grp.destroy()
    for _, _, _, o in outs:
        o.free()
    for _, dev in srcs:
        for d in dev.values():
            d.free()
    for l in lin.values():
        l.free()


def test_config5_three_planes_batch64_and_prefill(backend, oracle):
    """configs[4]: three additive planes (P(0)=0.4/0.7/0.85), hidden 5120, FFN 17408. Batch-64 decode of
    the up (K=5120) and down (K=17408, 68 K blocks) projections as single calls and as the grouped
    launch the benchmark times (8 x (up, down) members on the same weights), then the 4096-token
    prefill of both projections, and the one-plane 4096-token launch (4352 workgroups: the 4-tile form
    by itself). Every output against the exact composition; sampled tokens against the C oracle."""
    h, f = 5120, 17408
    rng = np.random.default_rng(5)
    shapes = {"up": (f, h), "down": (h, f)}
    host, lin = {}, {}
    for name, (n, k) in shapes.items():
        ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)]
        scs = [scales(rng, n) for _ in range(3)]
        packed = [T.pack_rows(w, n, k) for w in ws]
        host[name] = (ws, scs, packed)
        lin[name] = backend.linear(packed, scs, n, k)
    for m in (64, 4096):
        acts = {"up": _bf16(rng.standard_normal((m, h)).astype(np.float32)),
                "down": _bf16(rng.standard_normal((m, f)).astype(np.float32))}
        dev = {name: backend.to_device(bits, "bf16") for name, (bits, _) in acts.items()}
        want = {}
        for name, (n, k) in shapes.items():
            print("case config5", m, name, flush=True)
            ws, scs, packed = host[name]
            act = acts[name][1]
            want[name] = f32_to_bf16_bits(a8_expected(oracle, ws, scs, act)).reshape(m, n)
            tok = [0, m // 2 + 1, m - 1]
            ref = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act[tok], len(tok), n, k)
            assert (want[name][tok] == f32_to_bf16_bits(ref).reshape(len(tok), n)).all()
            o = backend.empty(m * n, "bf16")
            backend.linear_a8(lin[name], dev[name], m, o)
            assert (o.to_host().reshape(m, n) == want[name]).all()
            o.free()
        if m == 64:
            members, outs = [], []
            for _ in range(8):
                for name in ("up", "down"):
                    o = backend.empty(m * shapes[name][0], "bf16")
                    outs.append((name, o))
                    members.append((lin[name], dev[name], m, o))
            grp = backend.group(members, 1, "bf16", "bf16")
            grp.launch()
            grp.launch()
            for name, o in outs:
                assert (o.to_host().reshape(m, shapes[name][0]) == want[name]).all()
            grp.destroy()
            for _, o in outs:
                o.free()
        else:
            # one plane, 4096 tokens x 5120 -> 17408: raw int32 accumulators of every output
            n, k = shapes["up"]
            ws, scs, packed = host["up"]
            single = backend.linear([packed[0]], [scs[0]], n, k)
            q = rng.integers(-127, 128, (m, k)).astype(np.int8)
            dq, dacc = backend.to_device(q, "i8"), backend.empty(m * n, "i32")
            backend.linear_i8(single, dq, None, m, dacc)
            acc = dacc.to_host().reshape(m, n)
            exact = (q.astype(np.float32) @ np.ascontiguousarray(ws[0].T, np.float32)).astype(np.int32)
            assert (acc == exact).all()
            tok = [0, 2049, m - 1]
            assert (acc[tok] == oracle.int8_accumulators(packed[0], FMT_TQ2_0, q[tok], len(tok), n, k)).all()
            dq.free()
            dacc.free()
            single.free()
        for d in dev.values():
            d.free()
    for l in lin.values():
        l.free()


@pytest.mark.parametrize("m", [1, 2, 4, 8, 16])
def test_config2_sweep_full_layer(backend, oracle, m):
    """configs[1]: two planes (P(0)=0.4/0.7), K=2048, N=8192, bf16 activations, f32 out, every batch
    size of the sweep, as a grouped launch wide enough for the automatic kernel choice of the
    benchmark (32 copies of the layer). Float contract: 1e-3 of max|want| and the reference's
    1e-4*max(1,|want|) per output, every output of two copies."""
    n, k, copies = 8192, 2048, 32
    rng = np.random.default_rng(200 + m)
    ws = [ternary(rng, n, k, 0.4), ternary(rng, n, k, 0.7)]
    scs = [scales(rng, n), scales(rng, n)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    acts, members, outs = [], [], []
    for c in range(copies):
        bits, act = _bf16(rng.standard_normal((m, k)).astype(np.float32))
        d, o = backend.to_device(bits, "bf16"), backend.empty(m * n, "f32")
        acts.append((act, d))
        outs.append(o)
        members.append((layer, d, m, o))
    grp = backend.group(members, 0, "bf16", "f32")
    grp.launch()
    grp.launch()
    for c in (0, copies - 1):
        print("case config2-sweep", m, c, flush=True)
        got = outs[c].to_host().reshape(m, n)
        want = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, acts[c][0], m, n, k)
        assert rel_err(got, want) <= 1e-3
        assert accepts(got, want, rel=1e-4, floor=1.0).all()
    grp.destroy()
    for (_, d), o in zip(acts, outs):
        d.free()
        o.free()
    layer.free()


def test_config3_prefill_bf16_automatic_kernel(backend, oracle):
    """configs[2] exactly as the benchmark times it: 2048 bf16 tokens x 2560 -> 6912, one plane, W1.58A8,
    bf16 out, one tk_linear_a8 call with the automatic kernel choice -- which must be one of the wide-tile
    prefill kernels, not the 64-row form. Every output against the exact composition, sampled tokens of it
    against the C oracle (crates/tritium-cuda/src/cuda/tests.rs:2100-2190 holds the reference's GPU GEMM to
    its CPU backend the same way)."""
    rng = np.random.default_rng(33)
    m, n, k = 2048, 6912, 2560
    w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [sc], n, k)
    bits, act = _bf16(rng.standard_normal((m, k)).astype(np.float32))
    dact, dout = backend.to_device(bits, "bf16"), backend.empty(m * n, "bf16")
    print("case config3-bf16-auto", flush=True)
    backend.linear_a8(layer, dact, m, dout)
    took = backend.last_kernel()
    assert took in ("gemm128", "gemm256"), took
    want = a8_expected(oracle, [w], [sc], act)
    assert (dout.to_host().reshape(m, n) == f32_to_bf16_bits(want).reshape(m, n)).all()
    tok = [0, 1, 63, 64, 777, 1023, 1024, 2047]
    rc, ref = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act[tok], sc, len(tok), n, k)
    assert rc == 0 and same_bits(want[tok], ref)
    # f32 out through the same kernel: the oracle's bits themselves
    dout32 = backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout32)
    assert backend.last_kernel() == took
    got32 = dout32.to_host().reshape(m, n)
    assert same_bits(got32, want) and same_bits(got32[tok], ref)
    for b in (dact, dout, dout32):
        b.free()
    layer.free()


def test_config5_attention_projections_batch64_ksplit(backend, oracle):
    """configs[4]'s attention projections as single 64-token calls: q / o 5120 x 5120 and k / v 1024 x 5120,
    three planes (P(0)=0.4/0.7/0.85), bf16 in and out. 20 and 4 workgroups of the prefill kernel: the automatic
    K split. Every output against the C oracle's plane composition."""
    h, m = 5120, 64
    rng = np.random.default_rng(55)
    bits, act = _bf16(rng.standard_normal((m, h)).astype(np.float32))
    dact = backend.to_device(bits, "bf16")
    for name, n in (("q", 5120), ("k", 1024)):
        print("case config5-attn", name, flush=True)
        ws = [ternary(rng, n, h, p0) for p0 in (0.4, 0.7, 0.85)]
        scs = [scales(rng, n) for _ in range(3)]
        packed = [T.pack_rows(w, n, h) for w in ws]
        layer = backend.linear(packed, scs, n, h)
        o = backend.empty(m * n, "bf16")
        backend.linear_a8(layer, dact, m, o)
        assert backend.last_kernel() == "gemm64_ksplit", backend.last_kernel()
        ref = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, h)
        assert (o.to_host().reshape(m, n) == f32_to_bf16_bits(ref).reshape(m, n)).all()
        o32 = backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, o32)
        assert same_bits(o32.to_host(), ref)
        o.free()
        o32.free()
        layer.free()
    dact.free()
