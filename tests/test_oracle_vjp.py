"""Pins the oracle's mpgemm_projected_vjp: the reference's own known-answer case, a float64
evaluation of the three sums, the order of the f32 adds, and the error behaviour the reference's
tests fix (crates/tritium-cpu/src/lib.rs:496-700)."""
import numpy as np

from helpers import ternary
from oracle_lib import FMT_TQ1_0, FMT_TQ2_0

TO_ERR_SHAPE, TO_ERR_BACKEND = 1, 5


def test_reference_known_answer(oracle):
    """crates/tritium-cpu/src/lib.rs:500-533, every number from the reference's test."""
    w = np.array([[1, 0, -1], [-1, 1, 1]], np.int8)
    packed = oracle.pack_matrix(w, 2, 3, FMT_TQ2_0)
    rc, ga, gw, gb = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [1.0, 2.0, 3.0, -1.0, 4.0, 0.5], [2.0, 0.5],
                                              [3.0, -2.0, 4.0, 1.0], 2, 2, 3)
    assert rc == 0
    assert ga.reshape(-1).tolist() == [7.0, -1.0, -7.0, 7.5, 0.5, -7.5]
    assert gw.reshape(-1).tolist() == [-1.0, 22.0, 11.0, -3.0, 0.0, -5.5]
    assert gb.tolist() == [7.0, -1.0]


def test_matches_float64_sums(oracle):
    """The shapes of the reference's device test (crates/tritium-cuda/src/cuda/tests.rs:734) and its
    packed-decode test (lib.rs:535-598); a transposed operand, a dropped scale or a wrong reduction
    axis is far outside the f32 rounding of sums this short."""
    rng = np.random.default_rng(3)
    for fmt in (FMT_TQ2_0, FMT_TQ1_0):
        for m, n, k in ((2, 3, 5), (7, 4, 257), (1, 33, 64), (2, 3, 257)):
            w = ternary(rng, n, k)
            packed = oracle.pack_matrix(w, n, k, fmt)
            act = rng.uniform(-2, 2, (m, k)).astype(np.float32)
            sc = rng.uniform(0.05, 1.5, n).astype(np.float32)
            gy = rng.uniform(-1, 1, (m, n)).astype(np.float32)
            rc, ga, gw, gb = oracle.cpu_projected_vjp(packed, fmt, act, sc, gy, m, n, k)
            assert rc == 0
            p64 = w.astype(np.float64) * sc.astype(np.float64)[:, None]
            for got, want in ((ga, gy.astype(np.float64) @ p64), (gw, gy.astype(np.float64).T @ act.astype(np.float64)),
                              (gb, gy.astype(np.float64).sum(0))):
                assert np.abs(got - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_sums_run_in_index_order(oracle):
    """1 + 2^-24 + 2^-24 in f32 is 1 when added left to right and 1 + 2^-23 when the small terms meet
    first: the n order of grad_act and the m order of grad_w and grad_bias show in the last bit."""
    tiny = np.float32(2.0 ** -24)
    w = np.ones((3, 1), np.int8)
    packed = oracle.pack_matrix(w, 3, 1, FMT_TQ2_0)
    rc, ga, _, _ = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [1.0], [1.0, 1.0, 1.0], [1.0, tiny, tiny], 1, 3, 1)
    assert rc == 0 and ga[0, 0] == np.float32(1.0)
    rc, ga, _, _ = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [1.0], [1.0, 1.0, 1.0], [tiny, tiny, 1.0], 1, 3, 1)
    assert rc == 0 and ga[0, 0] == np.float32(1.0) + np.float32(2.0 ** -23)
    packed1 = oracle.pack_matrix(np.ones((1, 1), np.int8), 1, 1, FMT_TQ2_0)
    rc, _, gw, gb = oracle.cpu_projected_vjp(packed1, FMT_TQ2_0, [1.0, 1.0, 1.0], [1.0], [1.0, tiny, tiny], 3, 1, 1)
    assert rc == 0 and gw[0, 0] == np.float32(1.0) and gb[0] == np.float32(1.0)
    rc, _, gw, gb = oracle.cpu_projected_vjp(packed1, FMT_TQ2_0, [1.0, 1.0, 1.0], [1.0], [tiny, tiny, 1.0], 3, 1, 1)
    assert rc == 0 and gw[0, 0] == np.float32(1.0) + np.float32(2.0 ** -23) and gb[0] == gw[0, 0]


def test_products_are_rounded_before_the_sum(oracle):
    """upstream * (trit * scale) with the product rounded to f32 on its own: (1 + 2^-12)^2 needs 25
    bits, so a fused multiply-add into -(1 + 2^-11) leaves 2^-24 where the unfused form leaves 0."""
    a = np.float32(1.0 + 2.0 ** -12)
    packed = oracle.pack_matrix(np.array([[1], [-1]], np.int8), 2, 1, FMT_TQ2_0)
    rc, ga, _, _ = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [0.0], [a, np.float32(1.0 + 2.0 ** -11)], [a, 1.0], 1, 2, 1)
    assert rc == 0 and ga[0, 0] == 0.0


def test_reserved_code_is_refused_before_any_write(oracle):
    """lib.rs:600-638: byte 0 holds the logical trit, byte 1 only tail padding; either refuses."""
    for corrupt in (0, 1):
        packed = oracle.pack_matrix(np.ones((1, 1), np.int8), 1, 1, FMT_TQ2_0).copy()
        packed[corrupt] |= 3
        rc, ga, gw, gb = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [1.0], [1.0], [1.0], 1, 1, 1)
        assert rc == TO_ERR_BACKEND
        assert np.isnan(ga).all() and np.isnan(gw).all() and np.isnan(gb).all()


def test_zero_inner_dimension(oracle):
    """lib.rs:640-666: k = 0 still sums the bias."""
    rc, ga, gw, gb = oracle.cpu_projected_vjp(np.zeros(0, np.uint8), FMT_TQ2_0, [], [1.0, 2.0, 3.0],
                                              [1.0, 2.0, 3.0, -1.0, -2.0, -3.0], 2, 3, 0)
    assert rc == 0 and gb.tolist() == [0.0, 0.0, 0.0] and ga.size == 0 and gw.size == 0
    rc, _, _, gb = oracle.cpu_projected_vjp(np.zeros(0, np.uint8), FMT_TQ2_0, [], [1.0, 2.0, 3.0],
                                            [1.0, 2.0, 3.0, 1.0, 2.0, 4.0], 2, 3, 0)
    assert gb.tolist() == [2.0, 4.0, 7.0]


def test_bad_output_shape(oracle):
    """lib.rs:668-700."""
    packed = oracle.pack_matrix(np.ones((1, 1), np.int8), 1, 1, FMT_TQ2_0)
    rc, _, gw, _ = oracle.cpu_projected_vjp(packed, FMT_TQ2_0, [1.0], [1.0], [1.0], 1, 1, 1, bias=False, lens=(0, 1, 0))
    assert rc == TO_ERR_SHAPE and np.isnan(gw).all()
