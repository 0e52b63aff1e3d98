"""Pins the oracle's contraction, activation quant and fused fold.

Known answers are the reference's (crates/tritium-core/src/reference.rs:181-256,
crates/tritium-spec/src/lib.rs:458-478,568-594, crates/tritium-nn/src/ops/act_quant.rs:207-285,
crates/tritium-cpu/src/lib.rs:891-1003, kernel.rs:1069-1173).
"""
import numpy as np
import pytest

from oracle_lib import ERR_BACKEND, ERR_SHAPE, FMT_TQ1_0, FMT_TQ2_0


def test_zero_weights_give_zero_output(oracle):
    rc, out = oracle.reference_mpgemm([1, 2, 3, 4], [0, 0], [1.0], 2, 1, 2)
    assert rc == 0 and (out == 0).all()


def test_signs_add_and_subtract(oracle):
    rc, out = oracle.reference_mpgemm([10, 3, 5], [1, -1, 1], [2.0], 1, 1, 3)
    assert rc == 0 and out[0, 0] == 24.0


def test_shape_mismatch(oracle):
    rc, _ = oracle.reference_mpgemm([1, 2], [1, 1, 1], [1.0], 1, 1, 2)
    assert rc == ERR_SHAPE


def test_equals_float_matmul_small(oracle):
    """reference.rs:220-256 — add/sub/skip == matmul with the trit as a coefficient. Integer-valued
    tenths keep float64 matmul an independent exact-enough reference."""
    rng = np.random.default_rng(1)
    for _ in range(200):
        m, n, k = rng.integers(1, 4), rng.integers(1, 4), rng.integers(1, 8)
        act = ((rng.integers(0, 200, (m, k)) - 100) / 10).astype(np.float32)
        w = rng.integers(-1, 2, (n, k)).astype(np.int8)
        sc = ((rng.integers(0, 50, n) + 1) / 25).astype(np.float32)
        rc, got = oracle.reference_mpgemm(act, w, sc, m, n, k)
        want = (act.astype(np.float64) @ w.T.astype(np.float64)) * sc.astype(np.float64)
        assert rc == 0 and np.abs(got - want).max() < 1e-4


def test_exact_on_integers_transposition_sensitive(oracle):
    """Integer activations: every partial sum is exact, so the result must equal an integer matmul
    bit for bit. Non-square M,N,K make a transposed operand or swapped index fail."""
    rng = np.random.default_rng(2)
    m, n, k = 3, 5, 37
    act = rng.integers(-128, 128, (m, k)).astype(np.float32)
    w = rng.integers(-1, 2, (n, k)).astype(np.int8)
    sc = np.array([1, 2, 4, 8, 0.5], np.float32)
    rc, got = oracle.reference_mpgemm(act, w, sc, m, n, k)
    want = (act.astype(np.int64) @ w.T.astype(np.int64)).astype(np.float32) * sc
    assert rc == 0 and (got == want).all()


def test_k_order_single_f32_accumulator(oracle):
    """The fold is one f32 accumulator in k order: (1e8 + 1) - 1e8 == 0 in f32, while any pairwise
    or wider accumulation gives 1. A dropped `-` or a reordered sum fails this."""
    rc, out = oracle.reference_mpgemm([1e8, 1.0, 1e8], [1, 1, -1], [1.0], 1, 1, 3)
    assert rc == 0 and out[0, 0] == 0.0
    rc, out = oracle.reference_mpgemm([1.0, 1e8, 1e8], [1, 1, -1], [1.0], 1, 1, 3)
    assert rc == 0 and out[0, 0] == 0.0  # 1+1e8 rounds to 1e8 as well
    rc, out = oracle.reference_mpgemm([1e8, 1e8, 1.0], [1, -1, 1], [3.0], 1, 1, 3)
    assert rc == 0 and out[0, 0] == 3.0


def test_skip_means_skip(oracle):
    """A zero trit skips its activation entirely: NaN/Inf under a zero weight never reach the sum
    (reference.rs:44-48), under a non-zero weight they propagate (cpu lib.rs:982-1003)."""
    rc, out = oracle.reference_mpgemm([np.nan, 2.0, np.inf], [0, 1, 0], [1.0], 1, 1, 3)
    assert rc == 0 and out[0, 0] == 2.0
    rc, out = oracle.reference_mpgemm([np.nan, 2.0], [1, 1], [1.0], 1, 1, 2)
    assert np.isnan(out[0, 0])
    rc, out = oracle.reference_mpgemm([np.inf, 2.0], [-1, 1], [1.0], 1, 1, 2)
    assert out[0, 0] == -np.inf


# ---- activation quant --------------------------------------------------------------------

def test_act_quant_golden(oracle):
    q, s = oracle.quantize_act_int8([1.0, -2.0, 0.5, -0.5, 2.0, -1.0], 1, 6)
    assert q.tolist() == [[64.0, -127.0, 32.0, -32.0, 127.0, -64.0]]
    assert abs(s[0] - 2.0 / 127.0) < 1e-9
    assert s[0] == np.float32(2.0) / np.float32(127.0)


def test_act_quant_zero_row(oracle):
    q, s = oracle.quantize_act_int8([0.0, 0.0, 3.0, -6.0], 2, 2)
    assert q[0].tolist() == [0.0, 0.0] and s[0] == 0.0
    assert abs(s[1] - 6.0 / 127.0) < 1e-9


def test_act_quant_ties_to_even_table(oracle):
    # act_quant.rs:207-219 : γ = 127 makes s == 1, so v*s == v and only the rounding acts
    vals = [0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, 2.4999, 2.5001, 127.0]
    q, s = oracle.quantize_act_int8(vals, 1, len(vals))
    assert q[0].tolist() == [0, 2, 2, 4, 0, -2, -2, 2, 3, 127]
    assert s[0] == 1.0


def test_act_quant_single_element_and_saturation(oracle):
    q, s = oracle.quantize_act_int8([-3.5], 1, 1)  # act_quant.rs:276-285
    assert q[0, 0] == -127.0 and abs(s[0] - 3.5 / 127.0) < 1e-9
    q, _ = oracle.quantize_act_int8([-5.0, 5.0, -2.5, 1.25], 1, 4)
    assert q[0, 0] == -127.0 and q[0, 1] == 127.0


def test_act_quant_operation_order(oracle):
    """s = 127/γ is ONE f32 divide, then ONE f32 multiply, then ties-to-even (lib.rs:369-374).
    With γ = 0x3f0f475a and a = 0x3efdd71b, fl(127/γ) = 226.914367..., fl(a·s) = 112.5 exactly
    (checked with exact rationals) -> 112; the orders (a/γ)·127 and (a·127)/γ both give
    112.5000076 -> 113, and round-half-away would give 113 as well."""
    g = np.array([0x3F0F475A], np.uint32).view(np.float32)[0]
    a = np.array([0x3EFDD71B], np.uint32).view(np.float32)[0]
    q, s = oracle.quantize_act_int8([g, a, -a], 1, 3)
    assert q[0].tolist() == [127.0, 112.0, -112.0]
    assert s[0] == g / np.float32(127.0)


def test_act_quant_matches_numpy_random(oracle):
    # act_quant.rs:239-254 : xorshift rows in [-4, 4)
    rng = np.random.default_rng(3)
    act = (rng.random((7, 33), dtype=np.float32) * 8 - 4).astype(np.float32)
    q, s = oracle.quantize_act_int8(act, 7, 33)
    gamma = np.abs(act).max(axis=1)
    sc = (np.float32(127.0) / gamma).astype(np.float32)
    want = np.clip(np.rint((act * sc[:, None]).astype(np.float32)), -128, 127)
    assert (q == want).all()
    assert (s == (gamma / np.float32(127.0)).astype(np.float32)).all()
    assert ((q == np.trunc(q)) & (q >= -128) & (q <= 127)).all()


# ---- CPU backend composition ---------------------------------------------------------------

def test_fused_folds_per_token_scale(oracle):
    """spec lib.rs:568-594 : M=1,K=2,N=1, act [3,-1], w [1,-1], scale 2 -> 338·3/127."""
    t = np.zeros(256, np.int8)  # K padded to a block for the packed path
    t[0], t[1] = 1, -1
    act = np.zeros(256, np.float32)
    act[0], act[1] = 3.0, -1.0
    packed = oracle.pack_matrix(t, 1, 256, FMT_TQ2_0)
    rc, out = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act, [2.0], 1, 1, 256)
    assert rc == 0 and abs(out[0, 0] - 338.0 * 3.0 / 127.0) < 1e-5
    # exact association: ((float)acc * scale) * act_scale
    want = (np.float32(169.0) * np.float32(2.0)) * (np.float32(3.0) / np.float32(127.0))
    assert out[0, 0] == want


@pytest.mark.parametrize("fmt", [FMT_TQ2_0, FMT_TQ1_0])
def test_cpu_mpgemm_all_pos_neg_zero(oracle, fmt):
    # cpu lib.rs:891-980
    m, n, k = 2, 2, 256
    act = (np.arange(m * k) % 11 - 5).astype(np.float32).reshape(m, k)
    sc = np.ones(n, np.float32)
    for v, sign in ((1, 1.0), (-1, -1.0), (0, 0.0)):
        packed = oracle.pack_matrix(np.full(n * k, v, np.int8), n, k, fmt)
        rc, out = oracle.cpu_mpgemm(packed, fmt, act, sc, m, n, k)
        assert rc == 0
        for mi in range(m):
            assert (out[mi] == sign * act[mi].sum()).all()


def test_cpu_mpgemm_errors(oracle):
    packed = oracle.pack_matrix(np.zeros(256, np.int8), 1, 256, FMT_TQ2_0)
    # act too short for M=2 (cpu lib.rs:857-886)
    rc, _ = oracle.cpu_mpgemm(packed, FMT_TQ2_0, np.zeros(256), [1.0], 2, 1, 256, out_len=2)
    assert rc == ERR_SHAPE
    bad = packed.copy()
    bad[0] = 0x03
    rc, _ = oracle.cpu_mpgemm(bad, FMT_TQ2_0, np.zeros(256), [1.0], 1, 1, 256)
    assert rc == ERR_BACKEND


def test_ragged_k_matches_unpacked_reference(oracle):
    # tritium-nn/tests/layers.rs:138+ uses K=300; cuda tests use (1,7,300), (5,130,257)
    rng = np.random.default_rng(5)
    for (m, n, k) in [(1, 7, 300), (5, 13, 257), (3, 4, 1), (2, 3, 255)]:
        for fmt in (FMT_TQ2_0, FMT_TQ1_0):
            w = rng.integers(-1, 2, (n, k)).astype(np.int8)
            act = rng.standard_normal((m, k)).astype(np.float32)
            sc = rng.uniform(0.01, 0.1, n).astype(np.float32)
            packed = oracle.pack_matrix(w, n, k, fmt)
            rc, got = oracle.cpu_mpgemm(packed, fmt, act, sc, m, n, k)
            rc2, want = oracle.reference_mpgemm(act, w, sc, m, n, k)
            assert rc == 0 and rc2 == 0 and (got.view(np.uint32) == want.view(np.uint32)).all()


def test_int8_accumulators_equal_f32_fold(oracle):
    """|Σ| <= 128·K < 2^24: the int32 sum is the f32 fold's value (kernel.rs:588-599)."""
    rng = np.random.default_rng(6)
    for (m, n, k) in [(1, 5, 19), (2, 4, 512), (1, 8, 2560), (3, 3, 33)]:
        q = rng.integers(-128, 128, (m, k)).astype(np.int8)
        q[0, 0], q[0, -1] = -128, 127
        w = rng.integers(-1, 2, (n, k)).astype(np.int8)
        sc = (rng.integers(0, 50, n) / 25 + 0.1).astype(np.float32)
        packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
        acc = oracle.int8_accumulators(packed, FMT_TQ2_0, q, m, n, k)
        assert (acc == q.astype(np.int64) @ w.T.astype(np.int64)).all()
        rc, out = oracle.cpu_mpgemm(packed, FMT_TQ2_0, q.astype(np.float32), sc, m, n, k)
        assert rc == 0 and (out == acc.astype(np.float32) * sc).all()


def test_fast_baseline_is_bit_identical(oracle):
    """The timed SIMD/threaded baseline must equal the scalar oracle bit for bit
    (kernel.rs:1069-1173; determinism across thread counts cpu lib.rs:1073-1120)."""
    rng = np.random.default_rng(7)
    for (m, n, k) in [(3, 5, 19), (2, 4, 512), (1, 8, 2560), (3, 3, 33), (40, 6, 300)]:
        w = rng.integers(-1, 2, (n, k)).astype(np.int8)
        sc = (rng.integers(0, 50, n) / 25 + 0.1).astype(np.float32)
        packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
        fa = ((rng.integers(0, 20000, (m, k))) / 100 - 100).astype(np.float32)
        ia = rng.integers(-128, 128, (m, k)).astype(np.float32)
        for act, kinds in ((fa, (1, 2)), (ia, (3, 4))):
            rc, want = oracle.cpu_mpgemm(packed, FMT_TQ2_0, act, sc, m, n, k)
            for threads in (1, 4):
                got, used, kern = oracle.cpu_mpgemm_fast(packed, FMT_TQ2_0, act, sc, m, n, k, threads)
                assert (got.view(np.uint32) == want.view(np.uint32)).all()
                assert kern in kinds + (0,)
                assert 1 <= used <= threads


def test_planes_reduce_to_single_plane(oracle):
    rng = np.random.default_rng(8)
    m, n, k = 2, 6, 512
    w = rng.integers(-1, 2, (n, k)).astype(np.int8)
    sc = rng.uniform(0.01, 0.1, n).astype(np.float32)
    act = rng.standard_normal((m, k)).astype(np.float32)
    packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
    one = oracle.cpu_mpgemm_planes([packed], FMT_TQ2_0, [sc], act, m, n, k)
    rc, want = oracle.cpu_mpgemm(packed, FMT_TQ2_0, act, sc, m, n, k)
    assert (one.view(np.uint32) == want.view(np.uint32)).all()
    a8 = oracle.cpu_linear_a8_planes([packed], FMT_TQ2_0, [sc], act, m, n, k)
    rc, want = oracle.cpu_mpgemm_with_act_quant(packed, FMT_TQ2_0, act, sc, m, n, k)
    assert (a8.view(np.uint32) == want.view(np.uint32)).all()
    # two planes: linear in the planes
    w2 = rng.integers(-1, 2, (n, k)).astype(np.int8)
    sc2 = rng.uniform(0.01, 0.1, n).astype(np.float32)
    p2 = oracle.pack_matrix(w2, n, k, FMT_TQ2_0)
    two = oracle.cpu_mpgemm_planes([packed, p2], FMT_TQ2_0, [sc, sc2], act, m, n, k)
    rc, o2 = oracle.cpu_mpgemm(p2, FMT_TQ2_0, act, sc2, m, n, k)
    assert (two == one + o2).all()


def test_tolerance(oracle):
    # vector.rs:113-125 and its tests
    assert oracle.accepts(1.00005, 1.0)
    assert not oracle.accepts(1.001, 1.0)
    assert oracle.accepts(1000.05, 1000.0)       # relative to |want|
    assert oracle.accepts(0.00005, 0.0)          # floor 1
    assert not oracle.accepts(0.0002, 0.0)
    assert oracle.accepts(float("nan"), float("nan"))
    assert not oracle.accepts(1.0, float("nan"))
    assert oracle.accepts(float("inf"), float("inf"))
    assert not oracle.accepts(float("inf"), float("-inf"))
    assert not oracle.accepts(1e30, float("inf"))
    assert oracle.accepts(1.0, 1.0, bit_exact=True) and not oracle.accepts(1.0000001, 1.0, bit_exact=True)
    assert oracle.accepts(0.02, 0.0, floor=1000.0)  # accepts_with_floor


def test_bf16_helpers(oracle):
    assert oracle.f32_to_bf16(1.0) == 0x3F80
    assert oracle.bf16_to_f32(0x3F80) == 1.0
    # ties to even: 1 + 2^-8 is exactly between 1.0 and 1+2^-7 -> even mantissa (1.0)
    assert oracle.f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    assert oracle.f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82
    import torch
    x = torch.randn(1000, dtype=torch.float32)
    want = x.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    got = np.array([oracle.f32_to_bf16(v) for v in x.tolist()], np.uint16)
    assert (got == want).all()


# ---- RMSNorm (crates/tritium-nn/src/ops/rmsnorm.rs) ----

def test_rmsnorm_unit_weights(oracle):
    """The reference's own case (rmsnorm.rs:100-110): x = [3, 4], mean(x^2) = 12.5."""
    out = oracle.rmsnorm([3.0, 4.0], [1.0, 1.0], 0.0)
    inv = 1.0 / np.sqrt(np.float32(12.5))
    assert abs(out[0] - 3.0 * inv) < 1e-6 and abs(out[1] - 4.0 * inv) < 1e-6


def test_sum_squares_exact_on_small_integers(oracle):
    """Integer inputs whose squares sum below 2^24: every order gives the exact sum, so this pins
    the squaring and that every element of a ragged length is taken once."""
    rng = np.random.default_rng(3)
    for n in (1, 17, 255, 256, 257, 1000, 2559):
        x = rng.integers(-9, 10, n).astype(np.float32)
        assert oracle.sum_squares_canonical(x) == np.float32((x.astype(np.int64) ** 2).sum())


def test_sum_squares_folds_a_slot_before_the_tree(oracle):
    """x[1] and x[257] share slot 1: 1 + 1 = 2 survives next to 2^24 (2^24 + 2 is representable),
    where a sequential fold loses both ones to ties-to-even (2^24 + 1 -> 2^24 twice)."""
    x = np.zeros(258, np.float32)
    x[0], x[1], x[257] = 4096.0, 1.0, 1.0
    assert oracle.sum_squares_canonical(x) == np.float32(16777218.0)
    seq = np.float32(0.0)
    for v in x:
        seq = np.float32(seq + v * v)
    assert seq == np.float32(16777216.0)


def test_sum_squares_tree_pairs_slots_128_apart(oracle):
    """Slots 1 and 129 meet in the first tree step (off = 128) and reach slot 0 as 2; pairing
    neighbours, or folding the slots in order, would add each 1 to 2^24 on its own and lose it."""
    x = np.zeros(256, np.float32)
    x[0], x[1], x[129] = 4096.0, 1.0, 1.0
    assert oracle.sum_squares_canonical(x) == np.float32(16777218.0)
    y = np.zeros(256, np.float32)
    y[0], y[64], y[128] = 4096.0, 1.0, 1.0  # these meet 2^24 one at a time: both are lost
    assert oracle.sum_squares_canonical(y) == np.float32(16777216.0)


def test_rmsnorm_mean_eps_and_scale(oracle):
    n = 300
    # mean over n (not 256, not n-1): all 2.0 -> mean 4, inv 0.5 -> exactly 1.0
    assert (oracle.rmsnorm(np.full(n, 2.0), np.ones(n), 0.0) == 1.0).all()
    # eps sits inside the square root: mean 1, eps 3 -> 1/sqrt(4) = 0.5 (outside it would give 0.25)
    w = np.arange(n, dtype=np.float32)
    assert (oracle.rmsnorm(np.ones(n), w, 3.0) == np.float32(0.5) * w).all()
    # a zero row stays zero (eps keeps inv finite)
    assert (oracle.rmsnorm(np.zeros(n), w, 1e-5) == 0.0).all()
    # zero-centered: 0 is the identity scale, 1 doubles (rmsnorm.rs:55-63)
    assert (oracle.rmsnorm(np.full(n, 2.0), np.zeros(n), 0.0, zero_centered=True) == 1.0).all()
    assert (oracle.rmsnorm(np.full(n, 2.0), np.ones(n), 0.0, zero_centered=True) == 2.0).all()
    # n == 0 writes nothing
    assert oracle.rmsnorm(np.zeros(0), np.zeros(0), 1e-5).size == 0


def test_rmsnorm_multiplies_left_to_right(oracle):
    """out = (x * inv) * w, each product rounded (rmsnorm.rs:91-93): on a row where x * (inv * w)
    rounds differently the left-to-right value is the one returned."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal(512).astype(np.float32)
    w = rng.uniform(0.5, 1.5, 512).astype(np.float32)
    eps = np.float32(1e-5)
    inv = np.float32(1.0) / np.sqrt(np.float32(oracle.sum_squares_canonical(x) / np.float32(512) + eps))
    left = (x * inv) * w
    right = x * (inv * w)
    assert (left != right).any()
    assert (oracle.rmsnorm(x, w, eps).view(np.uint32) == left.view(np.uint32)).all()


def test_rmsnorm_quant_composes_and_zero_row(oracle):
    """Fused form = rmsnorm of each row, then quantize_act_int8 of it; an all-zero row gives zeros
    and scale 0 (crates/tritium-cuda/src/cuda/tests.rs:4759-4771)."""
    rng = np.random.default_rng(12)
    m, k = 3, 300
    x = rng.standard_normal((m, k)).astype(np.float32) * 3
    x[1] = 0.0
    w = rng.uniform(-2, 2, k).astype(np.float32)
    q, s = oracle.rmsnorm_quant(x, w, m, k, 1e-5)
    for r in range(m):
        qq, ss = oracle.quantize_act_int8(oracle.rmsnorm(x[r], w, 1e-5), 1, k)
        assert (q[r] == qq.reshape(-1)).all() and s[r] == ss[0]
    assert (q[1] == 0).all() and s[1] == 0.0
