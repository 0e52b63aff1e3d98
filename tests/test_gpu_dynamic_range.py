"""Float contract on heavy-tailed tokens: one or a few activations 2^12 .. 2^30 times the rest, placed
under zero and non-zero trits, f32 and bf16. Every output is graded on its own against the CPU
oracle's k-ordered f32 fold (crates/tritium-core/src/reference.rs:42-51) at the reference's
1e-4*max(1,|want|) (crates/tritium-testkit/src/vector.rs:113-125) and at a relative 1e-3. The fold
skips an activation under a zero trit, so such outputs are small next to the token's maximum: a
fixed-point grid laid against that maximum cannot carry them, and tokens of that kind must come out
of the reference-order path (bits equal the CPU's)."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, bf16_bits_to_f32, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def automatic_dispatch(backend):
    backend.set_decode_kernel(0)
    backend.set_flow_mfma(0)
    yield
    backend.set_decode_kernel(0)


def _per_output_ok(got, want, act, w, sc):
    """Per output: |got-want| <= 1e-4*max(1,|want|), and <= 1e-3*|want| wherever the output is not a
    cancellation (|want| at least 1e-3 of the sum of the magnitudes it adds up). `want` is the k-ordered
    f32 fold, which carries its own rounding (half an ulp of the running sum per step: visible where large
    terms cancel and leave a small output); an output that is closer to the exact value (float64) than the
    fold is passes too -- no method can agree with the fold better than the fold agrees with the truth."""
    exact = (act.astype(np.float64) @ w.T.astype(np.float64)) * sc.astype(np.float64)[None, :]
    cond = (np.abs(act).astype(np.float64) @ np.abs(w.T).astype(np.float64)) * sc[None, :]
    closer = np.abs(got - exact) <= np.abs(want - exact)
    ok4 = accepts(got, want, rel=1e-4, floor=1.0) | closer
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    graded = np.abs(want) >= 1e-3 * cond
    ok3 = ~graded | (diff <= 1e-3 * np.abs(want)) | closer
    return ok4, ok3, exact


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("spread", [12, 16, 20, 30])
@pytest.mark.parametrize("outliers", [1, 10])
def test_heavy_tailed_tokens_per_output(backend, oracle, dtype, spread, outliers):
    print("case heavy-tail", dtype, spread, outliers, flush=True)
    rng = np.random.default_rng(spread * 100 + outliers + (dtype == "bf16"))
    m, n, k = 6, 512, 2048
    w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    pos = rng.choice(k, outliers, replace=False)
    # tokens 0..3 carry the outliers (different signs and slightly different sizes), 4 and 5 stay plain
    for t in range(4):
        act[t, pos] = (2.0 ** spread) * (1.0 + 0.1 * t) * np.where(rng.random(outliers) < 0.5, -1.0, 1.0)
    # make sure both cases occur for the first outlier: a zero trit and a non-zero trit above it
    w[: n // 3, pos[0]] = 0
    w[n // 3: 2 * n // 3, pos[0]] = 1
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [sc], n, k)
    if dtype == "bf16":
        bits = f32_to_bf16_bits(act)
        act = bf16_bits_to_f32(bits).reshape(m, k)
        dact = backend.to_device(bits, "bf16")
    else:
        dact = backend.to_device(act, "f32")
    dout = backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    rc, want = oracle.cpu_mpgemm(packed, FMT_TQ2_0, act, sc, m, n, k)
    assert rc == 0
    ok4, ok3, exact = _per_output_ok(got, want, act, w, sc)
    assert ok4.all(), f"{(~ok4).sum()} outputs beyond 1e-4*max(1,|want|); worst token rows {np.unique(np.where(~ok4)[0])}"
    assert ok3.all(), f"{(~ok3).sum()} outputs beyond 1e-3*|want|"
    # against the exact value the kernel is within 1e-4*max(1,|exact|) wherever the fold is, and on the
    # plain tokens always
    tol = 1e-4 * np.maximum(1.0, np.abs(exact))
    assert (np.abs(got[4:] - exact[4:]) <= tol[4:]).all()
    assert ((np.abs(got - exact) <= tol) | (np.abs(want - exact) > tol)).all()
    if spread >= 20 or (dtype == "f32" and spread >= 16):
        # the grid cannot carry these tokens: they come out of the reference-order path, bit for bit
        # (bf16 elements down to 2^-6 still lie on the grid exactly at a spread of 2^16: those stay)
        assert same_bits(got[:4], want[:4])
    # the same through the prefill kernel's float path (more tokens than the decode kernels take)
    m2 = 20
    act2 = np.tile(act, (4, 1))[:m2]
    d2 = backend.to_device(f32_to_bf16_bits(act2) if dtype == "bf16" else act2, dtype)
    o2 = backend.empty(m2 * n, "f32")
    backend.linear_float(layer, d2, m2, o2)
    got2 = o2.to_host().reshape(m2, n)
    assert same_bits(got2[:m], got)  # every kernel finishes a token the same way
    for a in (dact, dout, d2, o2):
        a.free()
    layer.free()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_plain_and_integer_tokens_stay_on_the_fast_path(backend, oracle, dtype):
    """N(0,1) tokens, int8-valued tokens, and tokens with 200 large elements (every output meets some of
    them) are not sent to the reference-order path: the kernel's answer differs from the fold's in the
    last bits on N(0,1) input (if it were the exact path the bits would agree), and stays within both
    tolerances per output."""
    rng = np.random.default_rng(7 + (dtype == "bf16"))
    m, n, k = 5, 640, 2048
    w, sc = ternary(rng, n, k, 0.4), scales(rng, n)
    act = rng.standard_normal((m, k)).astype(np.float32)
    act[1] = rng.integers(-128, 128, k).astype(np.float32)           # what TernaryLinear feeds mpgemm
    big = rng.choice(k, 200, replace=False)
    act[2, big] *= 2.0 ** 20                                          # many large elements
    act[3, 5] = 0.0
    act[3] *= 1e-20                                                   # tiny overall scale: the grid follows it
    packed = T.pack_rows(w, n, k)
    layer = backend.linear([packed], [sc], n, k)
    if dtype == "bf16":
        bits = f32_to_bf16_bits(act)
        act = bf16_bits_to_f32(bits).reshape(m, k)
        dact = backend.to_device(bits, "bf16")
    else:
        dact = backend.to_device(act, "f32")
    dout = backend.empty(m * n, "f32")
    backend.linear_float(layer, dact, m, dout)
    got = dout.to_host().reshape(m, n)
    rc, want = oracle.cpu_mpgemm(packed, FMT_TQ2_0, act, sc, m, n, k)
    ok4, ok3, exact = _per_output_ok(got, want, act, w, sc)
    assert ok4.all() and ok3.all()
    assert same_bits(got[1], want[1])            # integers are exact on the grid
    assert not same_bits(got[0], want[0])        # the fixed-point answer, not the fold's rounding
    for t in (0, 2, 3, 4):                        # and it is the tighter of the two
        assert np.abs(got[t] - exact[t]).max() <= np.abs(want[t] - exact[t]).max() * 1.01 + 1e-30
    dact.free()
    dout.free()
    layer.free()
