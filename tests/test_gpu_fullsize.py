"""BASELINE-size checks: size-independent properties at full shapes plus sampled oracle rows."""
import numpy as np
import pytest

import tritium_amd as T
from helpers import accepts, rel_err, same_bits, scales, ternary
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
