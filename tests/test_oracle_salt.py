"""Pins the oracle's SALT restatement (block-scale additive planes): the f16 conversion against
numpy's, the dequantized row against an independent numpy statement, the one-plane unit-scale case
against the plain reference contraction (exact), and the plane order of the f32 sum."""
import numpy as np

from helpers import ternary
from oracle_lib import FMT_TQ2_0


def f16_bits(x):
    return np.asarray(x, np.float16).view(np.uint16)


def test_f16_to_f32_every_bit_pattern(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(b) for b in bits], np.float32)
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all()
    assert (got.view(np.uint32)[~nan] == want.view(np.uint32)[~nan]).all()


def test_dequant_row_matches_numpy_statement(oracle):
    """W[i] = sum_p f32(s_p[i // 256]) * t_p[i], planes added in order from 0.0 (salt.rs:720-738)."""
    rng = np.random.default_rng(31)
    for k, T in ((256, 1), (300, 2), (1000, 3)):
        nb = (k + 255) // 256
        trits = [ternary(rng, 1, k, 0.5)[0] for _ in range(T)]
        sc = [f16_bits(rng.uniform(0.01, 2.0, nb)) for _ in range(T)]
        rows = [oracle.pack_row(trits[p], FMT_TQ2_0, sc[p])[1] for p in range(T)]
        rc, w = oracle.salt_dequant_row(rows, k)
        assert rc == 0
        want = np.zeros(k, np.float32)
        for p in range(T):
            want = want + np.repeat(sc[p].view(np.float16).astype(np.float32), 256)[:k] * trits[p].astype(np.float32)
        assert (w.view(np.uint32) == want.view(np.uint32)).all()


def test_plane_order_of_the_sum(oracle):
    """(1 + 2^-11) - 1 in f32: planes (1, 2^-11... ) chosen so that the order of the f32 adds shows:
    2048 + 0.5 rounds to 2048 (f32 has 24 bits; f16 holds both scales exactly), then - 2048 gives 0;
    the other order, 2048 - 2048 + 0.5, gives 0.5."""
    k = 256
    t_pos, t_neg = np.ones(k, np.int8), -np.ones(k, np.int8)
    big, small = f16_bits([2048.0]), f16_bits([0.000061035156])  # 2^-14
    rows = [oracle.pack_row(t_pos, FMT_TQ2_0, big)[1], oracle.pack_row(t_pos, FMT_TQ2_0, small)[1],
            oracle.pack_row(t_neg, FMT_TQ2_0, big)[1]]
    rc, w = oracle.salt_dequant_row(rows, k)
    assert rc == 0 and (w == 0.0).all()          # (2048 + 2^-14) - 2048 = 0 in f32
    rc, w = oracle.salt_dequant_row([rows[0], rows[2], rows[1]], k)
    assert rc == 0 and (w == np.float32(2.0 ** -14)).all()


def test_one_plane_unit_scale_is_the_plain_contraction(oracle):
    rng = np.random.default_rng(32)
    m, n, k = 3, 7, 600
    w = ternary(rng, n, k)
    act = rng.standard_normal((m, k)).astype(np.float32)
    rc, out = oracle.salt_mpgemm([oracle.pack_matrix(w, n, k, FMT_TQ2_0)], n, k, act, m)
    rc2, want = oracle.reference_mpgemm(act, w, np.ones(n, np.float32), m, n, k)
    assert rc == 0 and rc2 == 0 and (out.view(np.uint32) == want.view(np.uint32)).all()


def test_forward_is_a_sequential_f32_dot_of_the_dequantized_row(oracle):
    rng = np.random.default_rng(33)
    m, n, k, T = 2, 5, 520, 2
    nb = 3
    trits = [ternary(rng, n, k, 0.4), ternary(rng, n, k, 0.7)]
    sc = [f16_bits(rng.uniform(0.05, 1.0, (n, nb))) for _ in range(T)]
    planes = [oracle.pack_matrix_scaled(trits[p], sc[p], n, k) for p in range(T)]
    act = rng.standard_normal((m, k)).astype(np.float32)
    rc, out = oracle.salt_mpgemm(planes, n, k, act, m)
    assert rc == 0
    for ni in range(n):
        w = np.zeros(k, np.float32)
        for p in range(T):
            w = w + np.repeat(sc[p][ni].view(np.float16).astype(np.float32), 256)[:k] * trits[p][ni].astype(np.float32)
        for mi in range(m):
            acc = np.float32(0.0)
            for ki in range(k):
                acc = np.float32(acc + np.float32(act[mi, ki] * w[ki]))
            assert out[mi, ni].view(np.uint32) == acc.view(np.uint32)
