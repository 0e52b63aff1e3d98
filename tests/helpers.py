"""Shared helpers for the parity tests: seeded synthetic inputs and bf16 bit conversions."""
import numpy as np

from oracle_lib import FMT_TQ1_0, FMT_TQ2_0  # noqa: F401


def f32_to_bf16_bits(x):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(h):
    return (np.ascontiguousarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def ternary(rng, n, k, p_zero=0.4):
    """i.i.d. trits with P(0)=p_zero, P(+1)=P(-1)."""
    u = rng.random((n, k))
    half = (1.0 - p_zero) / 2
    return np.where(u < p_zero, 0, np.where(u < p_zero + half, 1, -1)).astype(np.int8)


def scales(rng, n):
    return rng.uniform(0.01, 0.1, n).astype(np.float32)


def rel_err(got, want):
    """max |got-want| / max(1e-30, max|want|): the normalised error the float-path bound is stated in."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    return float(np.abs(got - want).max() / max(1e-30, np.abs(want).max()))


def accepts(got, want, rel=1e-4, floor=1.0):
    """Vectorised Tolerance::accepts_with_floor (crates/tritium-testkit/src/vector.rs:113-125)."""
    got = np.asarray(got, np.float32)
    want = np.asarray(want, np.float32)
    floor = np.broadcast_to(np.asarray(floor, np.float32), want.shape)
    nan = np.isnan(want) | np.isnan(got)
    inf = np.isinf(want) | np.isinf(got)
    ok = np.abs(got - want) <= np.float32(rel) * np.maximum(np.abs(want), floor)
    ok = np.where(inf, got == want, ok)
    ok = np.where(nan, np.isnan(want) & np.isnan(got), ok)
    return ok


def same_bits(a, b):
    a = np.ascontiguousarray(a, np.float32).reshape(-1)
    b = np.ascontiguousarray(b, np.float32).reshape(-1)
    return bool((a.view(np.uint32) == b.view(np.uint32)).all())


def a8_expected(oracle, ws, scs, act):
    """The W1.58A8 composition for whole tensors: quantize per token with the oracle, contract exactly
    (integer products summed in f32 BLAS: every partial sum is an integer below 2^24 for K <= 65536, so
    any summation order gives the exact value), then ((float)acc * s_w[n]) summed over planes in order,
    times the per-token scale -- every step one f32 rounding, as crates/tritium-cpu/src/kernel.rs:921-922
    and crates/tritium-nn/src/layers/linear.rs:272-277 do. Tests that use it also compare sampled rows
    with the C oracle, which pins this restatement."""
    m, k = act.shape
    assert k * 128 < (1 << 24)
    q, s = oracle.quantize_act_int8(act, m, k)
    qf = np.ascontiguousarray(q, np.float32).reshape(m, k)
    out = None
    for w, sc in zip(ws, scs):
        acc = qf @ np.ascontiguousarray(w.T, np.float32)
        t = acc * np.asarray(sc, np.float32)[None, :]
        out = t if out is None else out + t
    return (out * np.asarray(s, np.float32).reshape(m, 1)).astype(np.float32)
