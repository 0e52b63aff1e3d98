"""The entry point that allocates nothing (tk_linear_a8_noalloc, static device scratch) against
tk_linear_a8: identical bits, on calls in a row that share the scratch, the later ones smaller, and
a loud refusal beyond the scratch size. Collected last: a failure here must not hide other tests."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


def _layer(backend, rng, n, k, planes):
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    return packed, scs, backend.linear(packed, scs, n, k)


def test_noalloc_equals_linear_a8_on_consecutive_calls(backend, oracle):
    """A big call (prefill kernel, two planes), then smaller ones on the same scratch (decode kernels,
    other K, other plane count): what the earlier call left in the scratch must not leak into the later."""
    rng = np.random.default_rng(77)
    cases = [(200, 136, 2560, 2, "f32"), (40, 136, 2560, 2, "f32"), (3, 129, 700, 1, "bf16"), (1, 48, 300, 3, "f32"),
             (1, 8300, 512, 1, "bf16"), (4, 8300, 512, 2, "f32")]  # (wide layers: the flow kernel, in one launch for one token)
    for m, n, k, planes, dt in cases:
        print("case noalloc", m, n, k, planes, dt, flush=True)
        packed, scs, layer = _layer(backend, rng, n, k, planes)
        act = rng.standard_normal((m, k)).astype(np.float32)
        if m > 2:
            act[1] = 0.0
        if dt == "bf16":
            bits = f32_to_bf16_bits(act)
            act = (bits.astype(np.uint32) << 16).view(np.float32).reshape(m, k)
            dact = backend.to_device(bits, "bf16")
        else:
            dact = backend.to_device(act, "f32")
        d_ref, d_new = backend.empty(m * n, "f32"), backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, d_ref)
        backend.linear_a8_noalloc(layer, dact, m, d_new)
        ref, new = d_ref.to_host(), d_new.to_host()
        assert same_bits(new, ref)
        assert same_bits(new, oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k))
        for a in (dact, d_ref, d_new):
            a.free()
        layer.free()


def test_noalloc_refuses_beyond_the_scratch(backend):
    """2048 tokens x K=8192 needs 2064 * 32 * 256 bytes of operand rows = 16.9 MB > 8 MiB: a clear error,
    nothing launched."""
    rng = np.random.default_rng(78)
    m, n, k = 2048, 16, 8192
    _, _, layer = _layer(backend, rng, n, k, 1)
    dact, dout = backend.empty(m * k, "f32"), backend.empty(m * n, "f32")
    with pytest.raises(T.InvalidInput, match="static scratch"):
        backend.linear_a8_noalloc(layer, dact, m, dout)
    backend.linear_a8(layer, dact, 1, dout)  # the context still works
    backend.sync()
    for a in (dact, dout):
        a.free()
    layer.free()
