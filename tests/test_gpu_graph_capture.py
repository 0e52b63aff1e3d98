"""Calls of the library under HIP stream capture: once a call of the same shapes has run (the workspace has its size,
the arrival counters of the K-split kernels exist), a linear call enqueues kernels and event waits only -- no
allocation, no synchronization, no memset -- so a caller can capture its decode step into a graph and replay it.
Every replay is checked against the eager result, with eager calls of the library that overwrite the same outputs
between the replays."""
import ctypes as C

import numpy as np
import pytest

import tritium_amd as T
from helpers import f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


def _hip():
    return C.CDLL("libamdhip64.so.7")  # the runtime the library is linked against, already in the process


def _ok(rc, what):
    assert rc == 0, f"{what}: hip error {rc}"


def test_a_decode_step_replays_from_a_graph(backend, oracle):
    """One decoder layer's worth of dependent calls (a q,k,v group behind an RMSNorm, o, a gate,up group behind an
    RMSNorm, down) at 1 and at 20 tokens, a float-contract call and the entry point that allocates nothing: captured
    once, replayed three times."""
    hip = _hip()
    stream = C.c_void_p(backend.stream_handle())
    assert stream.value
    rng = np.random.default_rng(4242)
    h, f, kv = 512, 1280, 128
    shapes = {"q": (h, h), "k": (kv, h), "v": (kv, h), "o": (h, h), "gate": (f, h), "up": (f, h), "down": (h, f)}
    host = {name: (T.pack_rows(ternary(rng, n, k, 0.4), n, k), scales(rng, n)) for name, (n, k) in shapes.items()}
    lin = {name: backend.linear([host[name][0]], [host[name][1]], *shapes[name]) for name in shapes}
    nw = [backend.to_device(rng.uniform(0.5, 1.5, h).astype(np.float32), "f32") for _ in range(2)]
    for m in (1, 20):
        print("case graph capture", m, flush=True)
        src = {key: f32_to_bf16_bits(rng.standard_normal((m, kk)).astype(np.float32)) for key, kk in (("hid", h), ("att", h), ("mid", f))}
        other = backend.to_device(f32_to_bf16_bits(rng.standard_normal((m, f)).astype(np.float32)), "bf16")
        hid, att, mid = (backend.to_device(src[key], "bf16") for key in ("hid", "att", "mid"))
        out = {name: backend.empty(m * shapes[name][0], "bf16") for name in shapes}
        out_f, out_n = backend.empty(m * h, "f32"), backend.empty(m * h, "f32")
        qkv = backend.group([(lin[x], hid, m, out[x]) for x in "qkv"], 1, "bf16", "bf16", norms=[(nw[0], 1e-5, False)] * 3)
        gu = backend.group([(lin[x], hid, m, out[x]) for x in ("gate", "up")], 1, "bf16", "bf16", norms=[(nw[1], 1e-5, False)] * 2)

        def step():
            qkv.launch()
            backend.linear_a8(lin["o"], att, m, out["o"])
            gu.launch()
            backend.linear_a8(lin["down"], mid, m, out["down"])
            backend.linear_float(lin["o"], att, m, out_f)
            backend.linear_a8_noalloc(lin["o"], att, m, out_n)

        def snapshot():
            backend.sync()
            return [x.to_host().copy() for x in list(out.values()) + [out_f, out_n]]

        step()
        step()
        want = snapshot()
        act_att = (src["att"].astype(np.uint32) << 16).view(np.float32).reshape(m, h)
        assert same_bits(want[-1], oracle.cpu_linear_a8_planes([host["o"][0]], FMT_TQ2_0, [host["o"][1]], act_att, m, h, h))
        graph, gexec, count = C.c_void_p(), C.c_void_p(), C.c_size_t(0)
        _ok(hip.hipStreamBeginCapture(stream, 0), "hipStreamBeginCapture")
        try:
            step()
        finally:
            rc = hip.hipStreamEndCapture(stream, C.byref(graph))
        _ok(rc, "hipStreamEndCapture")
        _ok(hip.hipGraphGetNodes(graph, None, C.byref(count)), "hipGraphGetNodes")
        assert count.value >= 6
        _ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)), "hipGraphInstantiate")
        try:
            for replay in range(3):
                # eager calls in between: other inputs into the same outputs, and the workspace reused
                backend.linear_a8(lin["down"], other, m, out["down"])
                backend.linear_a8(lin["q"], att, m, out["q"])
                backend.linear_float(lin["o"], hid, m, out_f)
                backend.linear_a8_noalloc(lin["o"], hid, m, out_n)
                backend.sync()
                _ok(hip.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
                got = snapshot()
                for a, b in zip(got, want):
                    assert same_bits(a, b), ("replay", replay, m)
        finally:
            _ok(hip.hipGraphExecDestroy(gexec), "hipGraphExecDestroy")
            _ok(hip.hipGraphDestroy(graph), "hipGraphDestroy")
        step()  # the context works eagerly afterwards
        for a, b in zip(snapshot(), want):
            assert same_bits(a, b)
        qkv.destroy()
        gu.destroy()
        for x in list(out.values()) + [out_f, out_n, hid, att, mid, other]:
            x.free()
    for l in lin.values():
        l.free()
    for w in nw:
        w.free()
