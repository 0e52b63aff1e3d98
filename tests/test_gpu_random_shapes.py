"""Seeded random shapes through the automatic dispatch: whatever kernel the library picks for (m, n, k, planes,
output type) -- decode forms, the 64-row and 128-row prefill kernels, the K split -- the W1.58A8 result carries
the CPU oracle's bits and the float contract stays inside the reference's conformance tolerance. The shapes are
ragged on purpose (rows, columns and K that are no multiples of any tile), with an all-zero token in each."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, f32_to_bf16_bits, same_bits, scales, ternary
from oracle_lib import FMT_TQ2_0

pytestmark = pytest.mark.gpu


def _draw(rng):
    kind = rng.integers(0, 4)
    if kind == 0:    # decode: few tokens, wide layers
        m, n, k = int(rng.integers(1, 65)), int(rng.integers(1, 1200)), int(rng.integers(1, 1800))
    elif kind == 1:  # prefill: many tokens
        m, n, k = int(rng.integers(65, 420)), int(rng.integers(1, 700)), int(rng.integers(1, 900))
    elif kind == 2:  # long rows (operand rows beyond LDS, K split candidates)
        m, n, k = int(rng.integers(17, 70)), int(rng.integers(1, 160)), int(rng.integers(2500, 7000))
    else:            # aligned shapes, where the 16-byte output paths apply
        m, n, k = int(rng.integers(1, 40)) * 16, int(rng.integers(1, 40)) * 16, int(rng.integers(1, 6)) * 256
    return m, n, k, int(rng.integers(1, 4))


@pytest.mark.parametrize("seed", range(48))
def test_random_shape_a8_bits_and_float_tolerance(backend, oracle, seed):
    rng = np.random.default_rng(0xA8000 + seed)
    m, n, k, planes = _draw(rng)
    print("case random-shape", seed, m, n, k, planes, flush=True)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    act = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-2, 3)).astype(np.float32)
    act[m // 2] = 0.0
    dact = backend.to_device(act, "f32")
    want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, act, m, n, k)
    dout = backend.empty(m * n, "f32")
    backend.linear_a8(layer, dact, m, dout)
    assert same_bits(dout.to_host(), want)
    dob = backend.empty(m * n, "bf16")
    backend.linear_a8(layer, dact, m, dob)
    assert (dob.to_host() == f32_to_bf16_bits(want).reshape(-1)).all()
    if m >= 65 and planes == 1:  # both prefill tile heights where the shape allows the 128-row kernel
        for rows in (64, 128):
            backend.set_gemm_rows(rows)
            backend.linear_a8(layer, dact, m, dout)
            assert same_bits(dout.to_host(), want)
        backend.set_gemm_rows(0)
    # the float contract on the first tokens (the CPU fold of every output costs K steps)
    mf = min(m, 24)
    dof = backend.empty(mf * n, "f32")
    backend.linear_float(layer, dact, mf, dof)
    wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, act[:mf], mf, n, k)
    top = max(float(np.abs(wantf).max()), 1e-30)
    assert accepts(dof.to_host().reshape(mf, n), wantf, rel=1e-4, floor=top).all()
    for a in (dact, dout, dob, dof):
        a.free()
    layer.free()


@pytest.mark.parametrize("seed", range(16))
def test_random_wide_layer_few_tokens(backend, oracle, seed):
    """Layers of more than two tiles per CU (N > 8192) with 1..16 tokens: the shapes whose kernel the dispatch picks
    by layer width -- the flow kernel's single-launch form for one token, the flow kernel behind a prep launch for few
    rows of several planes, the K-split kernel otherwise. Bits of the CPU under the int8 contract, the reference's
    tolerance under the float contract, ragged N and K."""
    rng = np.random.default_rng(0xB1D00 + seed)
    m = int(rng.choice([1, 1, 2, 3, 4, 8, 12, 16]))
    n, k, planes = int(rng.integers(8200, 13000)), int(rng.integers(200, 800)), int(rng.integers(1, 4))
    if seed % 4 == 0:
        k = int(rng.integers(1, 4)) * 256  # whole K blocks: the single-launch forms apply
    print("case random-wide", seed, m, n, k, planes, flush=True)
    ws = [ternary(rng, n, k, p0) for p0 in (0.4, 0.7, 0.85)[:planes]]
    scs = [scales(rng, n) for _ in range(planes)]
    packed = [T.pack_rows(w, n, k) for w in ws]
    layer = backend.linear(packed, scs, n, k)
    act = (rng.standard_normal((m, k)) * 10.0 ** rng.integers(-2, 3)).astype(np.float32)
    if m > 2:
        act[m // 2] = 0.0
    for dt in ("f32", "bf16"):
        a = act if dt == "f32" else (f32_to_bf16_bits(act).astype(np.uint32) << 16).view(np.float32).reshape(m, k)
        dact = backend.to_device(a if dt == "f32" else f32_to_bf16_bits(act), dt)
        want = oracle.cpu_linear_a8_planes(packed, FMT_TQ2_0, scs, a, m, n, k)
        dout = backend.empty(m * n, "f32")
        backend.linear_a8(layer, dact, m, dout)
        assert same_bits(dout.to_host(), want), (dt, backend.last_kernel())
        mf = min(m, 3)
        dof = backend.empty(mf * n, "f32")
        backend.linear_float(layer, dact, mf, dof)
        wantf = oracle.cpu_mpgemm_planes(packed, FMT_TQ2_0, scs, a[:mf], mf, n, k)
        top = max(float(np.abs(wantf).max()), 1e-30)
        assert accepts(dof.to_host().reshape(mf, n), wantf, rel=1e-4, floor=top).all(), (dt, backend.last_kernel())
        for x in (dact, dout, dof):
            x.free()
    layer.free()
