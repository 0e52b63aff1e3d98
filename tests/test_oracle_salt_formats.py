"""Pins the oracle's SALT part (oracle/salt_oracle.c) against the known answers the reference's own tests hold:
crates/tritium-format/src/salt.rs (tests from line 760), sparse.rs (tests from line 484), salt_v2.rs (tests from
line 540), crates/tritium-cpu/src/salt_v2.rs (tests from line 790) -- golden bytes, every rejection case, the
cancellation-before-scale answer -- plus exhaustive code round trips and an independent float64 product."""
import numpy as np
import pytest

import salt_oracle_lib as S
from oracle_lib import FMT_TQ2_0

F16_EIGHTH = np.float16(0.125).view(np.uint16)


@pytest.fixture(scope="module")
def so():
    return S.load()


def lcg_trits(k, seed):
    """a deterministic ternary row (any fixed generator does: the checks are round trips and structure)"""
    rng = np.random.default_rng(seed)
    return rng.integers(-1, 2, k).astype(np.int8)


def tq2_row(oracle, trits, scale_bits):
    k = trits.size
    nb = (k + 255) // 256
    rc, row = oracle.pack_row(trits, FMT_TQ2_0, np.full(nb, scale_bits, np.uint16))
    assert rc == 0
    return row


def sparse_residual(oracle, k, stride):
    """salt.rs tests make_sparse_residual: every stride-th weight non-zero, signs alternating, scale 0.125"""
    t = np.zeros(k, np.int8)
    i = np.arange(0, k, stride)
    t[i] = np.where((i // stride) % 2 == 0, 1, -1)
    return tq2_row(oracle, t, F16_EIGHTH)


# ------------------------------------------------------------------ SALT rows
def test_legacy_v1_row_layout_stays_byte_stable(so):
    rc, packed = so.pack_salt_row(1, [np.full(66, 0xA5, np.uint8)])
    assert rc == 0 and bytes(packed[:10]) == b"TSLT\x01\x01\x01\0\0\0" and (packed[10:] == 0xA5).all() and packed.size == 76


def test_progressive_row_is_smaller_exact_and_prefix_loadable(so, oracle):
    k = 4096
    planes = [tq2_row(oracle, lcg_trits(k, 1), 0x3C00), sparse_residual(oracle, k, 64), sparse_residual(oracle, k, 2)]
    rc1, legacy = so.pack_salt_row(k, planes)
    rc2, prog = so.pack_progressive_salt_row(k, planes, 0.10)
    assert rc1 == 0 and rc2 == 0 and prog.size < legacy.size
    assert (prog[10], prog[15], prog[20]) == (0, 1, 0)  # dense base, sparse residual, dense residual
    assert so.packed_salt_row_len(prog) == (0, prog.size)
    assert so.packed_salt_row_len(np.concatenate([prog, legacy])) == (0, prog.size)  # walks concatenated rows
    for data in (prog, legacy):
        rc, kk, got = so.unpack_salt_row(data)
        assert rc == 0 and kk == k and len(got) == 3 and all((g == p).all() for g, p in zip(got, planes))
    for mp in (0, 1, 2, 3, 1 << 40):
        rc, kk, got = so.unpack_salt_row(prog, mp)
        assert rc == 0 and len(got) == min(3, mp) and all((g == p).all() for g, p in zip(got, planes))


def test_progressive_row_rejects_malformed_framing(so, oracle):
    k = 4096
    planes = [tq2_row(oracle, lcg_trits(k, 2), 0x3C00), sparse_residual(oracle, k, 64)]
    rc, packed = so.pack_progressive_salt_row(k, planes, 0.10)
    assert rc == 0 and packed[15] == 1
    bad = packed.copy(); bad[10] = 1
    assert so.unpack_salt_row(bad)[0] == S.SPARSE_BASE_PLANE
    bad = packed.copy(); bad[15] = 9
    assert so.unpack_salt_row(bad)[0] == S.INVALID_PLANE_TAG
    sparse_start = 10 + 2 * 5 + planes[0].size
    bad = packed.copy(); bad[sparse_start + 6: sparse_start + 10] = np.frombuffer(np.uint32(k - 1).tobytes(), np.uint8)
    assert so.unpack_salt_row(bad)[0] == S.WRONG_LEN
    assert so.unpack_salt_row(packed[:-1])[0] == S.WRONG_LEN
    assert so.unpack_salt_row(np.concatenate([packed, np.zeros(1, np.uint8)]))[0] == S.WRONG_LEN
    bad = packed.copy(); bad[:4] = np.frombuffer(b"XSLT", np.uint8)
    assert so.unpack_salt_row(bad)[0] == S.BAD_MAGIC
    bad = packed.copy(); bad[4] = 3
    assert so.unpack_salt_row(bad)[0] == S.UNSUPPORTED_VERSION
    assert so.unpack_salt_row(packed[:9])[0] == S.WRONG_LEN


def test_prefix_reader_validates_omitted_dense_payloads(so, oracle):
    planes = [tq2_row(oracle, lcg_trits(256, 3), 0x3C00)]
    rc, prog = so.pack_progressive_salt_row(256, planes, 0.10)
    prog[15] = 0xFF  # four reserved codes in the first payload byte
    assert so.unpack_salt_row(prog, 0)[0] == S.OUT_OF_RANGE
    rc, legacy = so.pack_salt_row(256, planes)
    legacy[10] = 0xFF
    assert so.unpack_salt_row(legacy, 0)[0] == S.OUT_OF_RANGE


def test_nonzero_partial_padding_stays_dense_and_sparse_never_larger(so, oracle):
    k = 257
    residual = sparse_residual(oracle, k, 64)
    residual[66 + 1] = (residual[66 + 1] & ~np.uint8(3)) | np.uint8(2)  # a +1 in the padding of the last block
    planes = [tq2_row(oracle, lcg_trits(k, 4), 0x3C00), residual]
    rc, prog = so.pack_progressive_salt_row(k, planes, 1.0)
    assert rc == 0 and prog[15] == 0
    rc, kk, got = so.unpack_salt_row(prog)
    assert rc == 0 and all((g == p).all() for g, p in zip(got, planes))
    k = 4096
    planes = [tq2_row(oracle, lcg_trits(k, 5), 0x3C00), sparse_residual(oracle, k, 12)]  # 8.3% dense: below 10%, above break-even
    rc, prog = so.pack_progressive_salt_row(k, planes, 0.10)
    rc2, legacy = so.pack_salt_row(k, planes)
    assert rc == 0 and prog[15] == 0 and prog.size == legacy.size + 2 * 5
    for bad in (np.nan, -0.01, 1.01, np.inf):
        assert so.pack_progressive_salt_row(k, planes, bad)[0] == S.INVALID_DENSITY


def test_pruned_row_and_reserved_code(so, oracle):
    rc, packed = so.pack_salt_row(300, [])
    assert rc == 0 and packed.size == 10 and so.unpack_salt_row(packed)[:2] == (0, 300) and so.unpack_salt_row(packed)[2] == []
    bad = tq2_row(oracle, lcg_trits(300, 6), 0x3C00)
    bad[70] |= 0xC0
    assert so.pack_salt_row(300, [bad])[0] == S.OUT_OF_RANGE


# ------------------------------------------------------------------ sparse plane
@pytest.mark.parametrize("k,stride", [(512, 7), (300, 5), (1024, 13), (1, 1), (256, 300)])
def test_sparse_plane_round_trips_to_identical_dense_bytes(so, oracle, k, stride):
    dense = sparse_residual(oracle, k, stride)
    rc, scales, idx, sign = so.sparse_from_tq2_0(dense, k)
    assert rc == 0 and idx.size == len(range(0, k, stride)) and (idx == np.arange(0, k, stride)).all()
    rc, back = so.sparse_to_tq2_0(k, scales, idx, sign)
    assert rc == 0 and (back == dense).all()
    rc, enc = so.pack_sparse_plane(k, scales, idx, sign)
    assert rc == 0 and enc.size == 14 + 2 * ((k + 255) // 256) + 4 * idx.size and bytes(enc[:6]) == b"TSSP\x01\x00"
    assert int.from_bytes(bytes(enc[6:10]), "little") == k and int.from_bytes(bytes(enc[10:14]), "little") == idx.size
    if idx.size > 1:  # the second entry is negative: sign in the top bit
        e1 = int.from_bytes(bytes(enc[14 + 2 * ((k + 255) // 256) + 4:][:4]), "little")
        assert e1 == (stride | 0x80000000)
    rc, k2, s2, i2, g2 = so.unpack_sparse_plane(enc)
    assert rc == 0 and k2 == k and (s2 == scales).all() and (i2 == idx).all() and (g2 == sign).all()


def test_sparse_plane_rejections(so, oracle):
    k = 512
    dense = sparse_residual(oracle, k, 7)
    rc, scales, idx, sign = so.sparse_from_tq2_0(dense, k)
    rc, enc = so.pack_sparse_plane(k, scales, idx, sign)
    bad = enc.copy(); bad[0] = ord("X")
    assert so.unpack_sparse_plane(bad)[0] == S.BAD_MAGIC
    bad = enc.copy(); bad[4] = 2
    assert so.unpack_sparse_plane(bad)[0] == S.UNSUPPORTED_VERSION
    assert so.unpack_sparse_plane(enc[:-1])[0] == S.WRONG_LEN
    assert so.unpack_sparse_plane(enc[:13])[0] == S.WRONG_LEN
    first = 14 + 2 * 2
    bad = enc.copy(); bad[first: first + 4] = np.frombuffer(np.uint32(k).tobytes(), np.uint8)
    assert so.unpack_sparse_plane(bad)[0] == S.OUT_OF_RANGE
    bad = enc.copy(); bad[first + 4: first + 8] = bad[first: first + 4]  # duplicate column
    assert so.unpack_sparse_plane(bad)[0] == S.NONCANONICAL_INDICES
    assert so.pack_sparse_plane(k, scales, idx[::-1], sign)[0] == S.NONCANONICAL_INDICES
    assert so.pack_sparse_plane(k, scales, idx, np.zeros_like(sign))[0] == S.OUT_OF_RANGE
    assert so.pack_sparse_plane(k, scales[:1], idx, sign)[0] == S.WRONG_LEN
    assert so.pack_sparse_plane(1 << 31, scales, idx, sign)[0] == S.ROW_TOO_LONG
    padded = sparse_residual(oracle, 257, 64)
    padded[66 + 1] = (padded[66 + 1] & ~np.uint8(3)) | np.uint8(2)
    assert so.sparse_from_tq2_0(padded, 257)[0] == S.NONZERO_PADDING


# ------------------------------------------------------------------ SALT V2 codecs
def test_v2_codec_known_answers(so):
    assert bytes(so.v2_pack(S.D2, [-1, 0, 1, -1, 1])[1]) == b"\x24\x56"
    assert bytes(so.v2_pack(S.B3, [-1, 0, 1, -1, 1, 1])[1]) == b"\xb7\x7a"
    assert bytes(so.v2_pack(S.S34, [-1, 0, 1, -1, 1, -1, 0, 1])[1]) == b"\xc9\x02"
    for codec, t in ((S.D2, [-1, 0, 1, -1, 1]), (S.B3, [-1, 0, 1, -1, 1, 1]), (S.S34, [-1, 0, 1, -1, 1, -1, 0, 1])):
        rc, p = so.v2_pack(codec, t)
        rc, back = so.v2_unpack(codec, p, len(t))
        assert rc == 0 and list(back) == t
    # ledgers: salt_v2.rs tests d2_/b3_/s34_byte_ledger_is_exact
    assert so.v2_payload_bytes(S.D2, 5) == (0, 2) and so.v2_payload_bytes(S.B3, 6) == (0, 2) and so.v2_payload_bytes(S.S34, 12) == (0, 2)


def test_v2_codec_rejections(so):
    u = lambda *b: np.array(b, np.uint8)
    assert so.v2_unpack(S.D2, u(0b01010111), 1)[0] == S.V2_INVALID_D2_CODE
    assert so.v2_unpack(S.D2, u(0x00), 1)[0] == S.V2_NONCANONICAL_TRIT_PADDING
    assert so.v2_unpack(S.D2, u(0x55), 5)[0] == S.V2_WRONG_PACKED_LENGTH
    assert so.v2_unpack(S.B3, u(243), 5)[0] == S.V2_INVALID_B3_CODE
    assert so.v2_unpack(S.B3, u(0), 1)[0] == S.V2_NONCANONICAL_TRIT_PADDING
    assert so.v2_unpack(S.B3, u(121, 121), 1)[0] == S.V2_WRONG_PACKED_LENGTH
    assert so.v2_pack(S.S34, [1, 1, 1, 1])[0] == S.V2_S34_ZERO_COUNT
    assert so.v2_pack(S.S34, [0, 0, 1, 1])[0] == S.V2_S34_ZERO_COUNT
    assert so.v2_unpack(S.S34, u(0xC9, 0x82), 8)[0] == S.V2_NONCANONICAL_BIT_PADDING
    assert so.v2_unpack(S.S34, u(0xC9), 8)[0] == S.V2_WRONG_PACKED_LENGTH
    assert so.v2_pack(S.S34, [1, 0, 1])[0] == S.V2_S34_NOT_MULTIPLE_OF_FOUR


def test_every_b3_and_s34_code_is_canonical_and_round_trips(so):
    for code in range(243):
        rc, t = so.v2_unpack(S.B3, np.array([code], np.uint8), 5)
        assert rc == 0 and so.v2_pack(S.B3, t)[1][0] == code
        digits = [(code // 3 ** i) % 3 - 1 for i in range(5)]  # first trit in the least significant place
        assert list(t) == digits
    for code in range(32):
        rc, t = so.v2_unpack(S.S34, np.array([code], np.uint8), 4)
        assert rc == 0 and so.v2_pack(S.S34, t)[1][0] == code and (t == 0).sum() == 1 and t[code & 3] == 0


# ------------------------------------------------------------------ SALT V2 matrix-vector product
def test_v2_cancellation_happens_before_the_scale_and_overflow_is_rejected(so):
    fmax16 = np.float16(65504).view(np.uint16)
    fmax = np.float32(np.finfo(np.float32).max)
    t = S.V2Tensor(so, S.D2, 128, 1, 2, [(np.array([[1, -1]], np.int8), np.array([[fmax16]], np.uint16))])
    rc, out = so.v2_forward(t, np.array([fmax, fmax], np.float32), 1)
    assert rc == 0 and out[0, 0] == 0.0
    t = S.V2Tensor(so, S.D2, 128, 1, 2, [(np.array([[1, 1]], np.int8), np.array([[0x3C00]], np.uint16))])
    rc, out = so.v2_forward(t, np.array([fmax, fmax], np.float32), 1)
    assert rc == S.V2_NONFINITE_OUTPUT and out[0, 0] == np.float32(19.0)  # nothing stored
    t = S.V2Tensor(so, S.D2, 128, 1, 1, [(np.array([[1]], np.int8), np.array([[fmax16]], np.uint16))])
    rc, out = so.v2_forward(t, np.array([fmax], np.float32), 1)
    assert rc == S.V2_NONFINITE_OUTPUT and out[0, 0] == np.float32(19.0)
    rc, out = so.v2_forward(t, np.array([np.nan], np.float32), 1)
    assert rc == S.V2_NONFINITE_ACTIVATION and out[0, 0] == np.float32(19.0)


@pytest.mark.parametrize("codec", [S.D2, S.B3, S.S34])
@pytest.mark.parametrize("n,k,counts,group", [(3, 173, [1, 3, 2], 128), (5, 173, [1, 3, 2, 3], 128), (4, 256, None, 128),
                                               (7, 100, None, 64), (2, 1024, None, 128), (1, 4, [1], 128)])
def test_v2_forward_matches_independent_dense_math(so, codec, n, k, counts, group):
    if codec == S.S34 and (n * k) % 4:
        n += (4 - (n * k) % 4)  # S34 needs whole groups of four in the last tile
        counts = None
    if counts is not None and len(counts) != (n * k + 255) // 256:
        counts = None
    rng = np.random.default_rng(codec * 1000 + n * 10 + k)
    t = S.random_v2_tensor(so, rng, codec, n, k, counts, group)
    m = 2
    act = rng.uniform(-0.75, 0.75, (m, k)).astype(np.float32)
    rc, out = so.v2_forward(t, act, m)
    want = act.astype(np.float64) @ t.dense().T
    assert rc == 0 and np.abs(out - want).max() <= 1e-4 * max(1.0, np.abs(want).max())
    dense = t.dense()
    for index in {0, 127, 128, 255, 256, n * k - 1, n * k // 2} - {x for x in (127, 128, 255, 256) if x >= n * k}:
        rc, v = so.v2_coefficient(t, index)
        assert rc == 0 and abs(float(v) - dense.reshape(-1)[index]) <= 1e-6 * max(1.0, abs(dense.reshape(-1)[index]))
    assert so.v2_coefficient(t, n * k)[0] == S.OUT_OF_RANGE


def test_v2_forward_order_is_group_then_plane_then_column(so):
    """One row of two scale groups and two planes, values chosen so that every other association rounds
    differently: the answer must be ((g0p0*s + g0p1*s) + g1p0*s) + g1p1*s with each g a left-to-right f32 fold."""
    rng = np.random.default_rng(11)
    k = 256
    trits = rng.choice([-1, 1], (2, k)).astype(np.int8)
    sc = rng.uniform(0.5, 1.5, (2, 2)).astype(np.float16)
    t = S.V2Tensor(so, S.D2, 128, 1, k, [(trits, sc.view(np.uint16))])
    act = (rng.standard_normal(k) * 10.0 ** rng.integers(-3, 4, k)).astype(np.float32)
    rc, out = so.v2_forward(t, act.reshape(1, k), 1)
    acc = np.float32(0)
    for g in range(2):
        for p in range(2):
            ga = np.float32(0)
            for c in range(g * 128, (g + 1) * 128):
                ga = np.float32(ga + act[c]) if trits[p, c] > 0 else np.float32(ga - act[c])
            acc = np.float32(acc + np.float32(ga * np.float32(sc[p, g])))
    assert rc == 0 and out[0, 0].view(np.uint32) == acc.view(np.uint32)
