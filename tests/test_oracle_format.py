"""Pins the oracle's TQ2_0 / TQ1_0 restatement.

Golden bytes are the reference's own (crates/tritium-format/src/tq2.rs:215-241,
tq1.rs:133-150); round-trip sizes are rows.rs:210-240. The remaining checks use an
independent statement of each layout (closed forms / brute force), not the oracle's formula.
"""
import itertools

import numpy as np
import pytest

from oracle_lib import ERR_BACKEND, ERR_SHAPE, F16_ONE, FMT_TQ1_0, FMT_TQ2_0


def test_constants(oracle):
    # crates/tritium-format/src/lib.rs:144-150
    assert oracle.row_bytes(256, FMT_TQ2_0) == 66
    assert oracle.row_bytes(256, FMT_TQ1_0) == 54
    # rows.rs:226-233
    assert [oracle.num_blocks(k) for k in (0, 1, 256, 257, 4096)] == [0, 1, 1, 2, 16]
    # BASELINE shapes: K=2560 -> 660 B, K=2048 -> 528 B per row
    assert oracle.row_bytes(2560, FMT_TQ2_0) == 660
    assert oracle.row_bytes(2048, FMT_TQ2_0) == 528
    assert oracle.row_bytes(2560, FMT_TQ1_0) == 540


@pytest.mark.parametrize("v,byte", [(0, 0x55), (1, 0xAA), (-1, 0x00)])
def test_tq2_golden_bytes(oracle, v, byte):
    out = oracle.pack_block(np.full(256, v, np.int8), FMT_TQ2_0)
    assert (out[:64] == byte).all()
    assert bytes(out[64:]) == F16_ONE.to_bytes(2, "little")  # tq2.rs:220-222


@pytest.mark.parametrize("v,qs,qh", [(0, 0x80, 0x7F), (1, 0xFF, 0xFD), (-1, 0x00, 0x00)])
def test_tq1_golden_bytes(oracle, v, qs, qh):
    out = oracle.pack_block(np.full(256, v, np.int8), FMT_TQ1_0)
    assert (out[:48] == qs).all()
    assert (out[48:52] == qh).all()
    assert bytes(out[52:]) == F16_ONE.to_bytes(2, "little")


def test_unpack_golden_zero(oracle):
    b = np.full(66, 0x55, np.uint8)
    b[64:] = [0x00, 0x3C]
    rc, t, s = oracle.unpack_block(b, FMT_TQ2_0)
    assert rc == 0 and (t == 0).all() and s == F16_ONE
    b = np.zeros(54, np.uint8)
    b[:48] = 0x80
    b[48:52] = 0x7F
    b[52:] = [0x00, 0x3C]
    rc, t, s = oracle.unpack_block(b, FMT_TQ1_0)
    assert rc == 0 and (t == 0).all() and s == F16_ONE


def test_tq2_layout_independent(oracle):
    """Each element lands in exactly the byte/slot the format documents (tq2.rs:15-18):
    set one element at a time and look at which bit pair moved."""
    base = oracle.pack_block(np.zeros(256, np.int8), FMT_TQ2_0)[:64]
    for e in range(256):
        t = np.zeros(256, np.int8)
        t[e] = 1
        out = oracle.pack_block(t, FMT_TQ2_0)[:64]
        diff = np.nonzero(out != base)[0]
        c, rem = divmod(e, 128)
        n, m = divmod(rem, 32)
        assert list(diff) == [c * 32 + m]
        assert (out[c * 32 + m] >> (2 * n)) & 3 == 2
        assert out[c * 32 + m] == (0x55 & ~(3 << (2 * n))) | (2 << (2 * n))


def test_tq2_all_byte_contents(oracle):
    """Brute force over all 3^4 contents of one byte: numeric value == Σ (trit+1)·4^slot."""
    for combo in itertools.product((-1, 0, 1), repeat=4):
        t = np.zeros(256, np.int8)
        for n, v in enumerate(combo):
            t[n * 32 + 5] = v
        out = oracle.pack_block(t, FMT_TQ2_0)
        assert out[5] == sum((v + 1) << (2 * n) for n, v in enumerate(combo))
        rc, back, _ = oracle.unpack_block(out, FMT_TQ2_0)
        assert rc == 0 and (back == t).all()


def test_tq2_reserved_code_rejected(oracle):
    b = np.full(66, 0x55, np.uint8)
    b[10] = 0x57  # slot 0 holds code 3 -> trit 2
    rc, _, _ = oracle.unpack_block(b, FMT_TQ2_0)
    assert rc == ERR_BACKEND


def _tq1_independent_decode(block):
    """ggml's TQ1_0 stated from the number it encodes: byte q = ceil(v·256/243) with v the
    base-3 number (most significant digit first), so v = floor(q·243/256)."""
    t = np.zeros(256, np.int8)
    for m in range(32):
        v = (int(block[m]) * 243) // 256
        digs = [(v // 3 ** (4 - n)) % 3 for n in range(5)]
        for n in range(5):
            t[n * 32 + m] = digs[n] - 1
    for m in range(16):
        v = (int(block[32 + m]) * 243) // 256
        for n in range(5):
            t[160 + n * 16 + m] = (v // 3 ** (4 - n)) % 3 - 1
    for j in range(4):
        v = (int(block[48 + j]) * 243) // 256
        for n in range(4):
            t[240 + n * 4 + j] = (v // 3 ** (4 - n)) % 3 - 1
    return t


def test_tq1_all_groups_roundtrip(oracle):
    """All 3^5 groups through qs[0..32) and qs[32..48), all 3^4 through qh: decode∘encode = id,
    and the independent decoder agrees."""
    groups = list(itertools.product((-1, 0, 1), repeat=5))
    for start in range(0, 243, 32):
        t = np.zeros(256, np.int8)
        for m, g in enumerate(groups[start:start + 32]):
            for n in range(5):
                t[n * 32 + m] = g[n]
        for m, g in enumerate(groups[start:start + 16]):
            for n in range(5):
                t[160 + n * 16 + m] = g[4 - n]
        out = oracle.pack_block(t, FMT_TQ1_0)
        rc, back, _ = oracle.unpack_block(out, FMT_TQ1_0)
        assert rc == 0 and (back == t).all()
        assert (_tq1_independent_decode(out) == t).all()
    g4 = list(itertools.product((-1, 0, 1), repeat=4))
    for start in range(0, 81, 4):
        t = np.zeros(256, np.int8)
        for j, g in enumerate(g4[start:start + 4]):
            for n in range(4):
                t[240 + n * 4 + j] = g[n]
        out = oracle.pack_block(t, FMT_TQ1_0)
        rc, back, _ = oracle.unpack_block(out, FMT_TQ1_0)
        assert rc == 0 and (back == t).all()
        assert (_tq1_independent_decode(out) == t).all()


@pytest.mark.parametrize("fmt", [FMT_TQ2_0, FMT_TQ1_0])
@pytest.mark.parametrize("k", [1, 255, 256, 257, 4096])
def test_row_roundtrip_boundary_ks(oracle, fmt, k):
    rng = np.random.default_rng(k * 7 + fmt)
    t = rng.integers(-1, 2, size=k).astype(np.int8)
    nb = oracle.num_blocks(k)
    sc = (0x3C00 + np.arange(nb)).astype(np.uint16)
    rc, packed = oracle.pack_row(t, fmt, sc)
    assert rc == 0 and packed.size == nb * (66 if fmt == FMT_TQ2_0 else 54)
    rc, back, sc2 = oracle.unpack_row(packed, k, fmt)
    assert rc == 0 and (back == t).all() and (sc2 == sc).all()
    # a row is the concatenation of its blocks, the tail zero-padded (rows.rs:5-12)
    bb = packed.size // nb
    pad = np.zeros(nb * 256, np.int8)
    pad[:k] = t
    for i in range(nb):
        blk = oracle.pack_block(pad[i * 256:(i + 1) * 256], fmt, int(sc[i]))
        assert (blk == packed[i * bb:(i + 1) * bb]).all()


def test_partial_block_pads_with_zeros(oracle):
    # rows.rs:236-250
    t = np.ones(257, np.int8)
    t[256] = -1
    rc, packed = oracle.pack_row(t, FMT_TQ2_0)
    assert rc == 0
    rc, back, _ = oracle.unpack_row(packed, 257, FMT_TQ2_0)
    assert rc == 0 and (back == t).all()
    # block 1: element 0 is -1 (code 0 in slot 0 of byte 0), everything else code 1
    assert packed[66] == 0x54 and (packed[67:66 + 64] == 0x55).all()


def test_row_wrong_lengths(oracle):
    t = np.zeros(256, np.int8)
    rc, _ = oracle.pack_row(t, FMT_TQ2_0, np.array([F16_ONE, F16_ONE], np.uint16))
    assert rc == ERR_SHAPE  # rows.rs:252-262
    rc, _, _ = oracle.unpack_row(np.zeros(65, np.uint8), 256, FMT_TQ2_0)
    assert rc == ERR_SHAPE


def test_upload_check(oracle):
    # crates/tritium-cpu/src/lib.rs:801-813 : one byte short -> InvalidInput
    from oracle_lib import ERR_FORMAT, ERR_INVALID
    short = np.zeros(2 * 66 - 1, np.uint8)
    assert oracle.upload_check(short, 2, 256, FMT_TQ2_0)[0] == ERR_INVALID
    good = np.full(2 * 66, 0x55, np.uint8)
    assert oracle.upload_check(good, 2, 256, FMT_TQ2_0) == (0, -1)
    good[66 + 3] = 0xFF
    assert oracle.upload_check(good, 2, 256, FMT_TQ2_0) == (0, 1)
    assert oracle.upload_check(good, 2, 256, 7)[0] == ERR_FORMAT
