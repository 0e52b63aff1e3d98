"""Pins the oracle's I2_S restatement with the reference's own vectors
(crates/tritium-format/src/i2s.rs:160-334): a hand-built block, the striping of the four groups, the
first block of `blk.0.attn_q.weight` of the official BitNet GGUF with the trits the reference holds
for it, the reserved code, the length errors, the trailing scale; and pins the product's host
converter to the oracle."""
import numpy as np
import pytest

import tritium_amd as T
from oracle_lib import ERR_INVALID, ERR_SHAPE, FMT_TQ2_0

# i2s.rs:225-243 : the real block and its trits
REAL_BLOCK = bytes([
    0x42, 0x48, 0x61, 0x29, 0x55, 0x12, 0x44, 0x55, 0x55, 0x19, 0x54, 0x4a, 0xa1, 0x55,
    0x65, 0x51, 0x15, 0x51, 0x19, 0x55, 0x60, 0x51, 0x41, 0x44, 0x56, 0x55, 0x55, 0x14,
    0x51, 0x06, 0x45, 0x45])
REAL_TRITS = [
    0, 0, 0, -1, 0, -1, 0, 0, 0, -1, 0, 0, 1, 0, 0, 0, -1, 0, -1, 0, 0, 0, 0, 0, 0, 0, 0,
    -1, 0, -1, 0, 0, -1, -1, 1, 1, 0, 0, -1, 0, 0, 0, 0, -1, 1, 0, 1, 0, 0, 0, 0, 0, 1, 0,
    -1, -1, 0, 0, 0, 0, 0, -1, -1, -1, -1, 1, -1, 1, 0, -1, 0, 0, 0, 1, 0, 1, -1, 0, 0, -1,
    0, -1, 1, 0, -1, -1, -1, 0, 0, 0, 0, 0, -1, 0, 0, 0, 1, -1, 0, 0, 0, 1, -1, 0, 0, 0,
    -1, 1, 0, 0, 0, 0, 0, 0, 0, 0, -1, 0, 0, -1, 1, 0, 0, -1, 0, 1, 0, 0]


def i2s_payload(trits, scale, pad=0):
    """Independent statement of the layout (i2s.rs:1-4): element p of a 128-block sits in byte p % 32
    at bits 6 - 2*(p // 32); then the f32 scale; then `pad` bytes of GGUF alignment."""
    t = np.asarray(trits, np.int8).reshape(-1)
    assert t.size % 128 == 0
    q = np.zeros(t.size // 4, np.uint8)
    for i, v in enumerate(t):
        blk, p = divmod(i, 128)
        q[blk * 32 + p % 32] |= (int(v) + 1) << (6 - 2 * (p // 32))
    return np.concatenate([q, np.frombuffer(np.float32(scale).tobytes(), np.uint8), np.zeros(pad, np.uint8)])


def test_hand_golden_block(oracle):
    """i2s.rs:175-203"""
    block = np.full(32, 0b01010101, np.uint8)
    block[0], block[1] = 0b10010100, 0b01100001
    rc, t = oracle.unpack_i2s_block(block)
    assert rc == 0
    want = np.zeros(128, np.int8)
    want[0], want[96], want[33], want[65] = 1, -1, 1, -1
    assert (t == want).all()


def test_codes_stripe_each_position(oracle):
    """i2s.rs:205-222 : groups 0..3 hold codes 2, 0, 1, 2."""
    block = np.full(32, (0b10 << 6) | (0b00 << 4) | (0b01 << 2) | 0b10, np.uint8)
    rc, t = oracle.unpack_i2s_block(block)
    assert rc == 0
    assert (t[:32] == 1).all() and (t[32:64] == -1).all() and (t[64:96] == 0).all() and (t[96:] == 1).all()


def test_real_block_from_the_bitnet_gguf(oracle):
    """i2s.rs:224-252"""
    rc, t = oracle.unpack_i2s_block(np.frombuffer(REAL_BLOCK, np.uint8))
    assert rc == 0 and t.tolist() == REAL_TRITS


def test_block_errors(oracle):
    """i2s.rs:254-290"""
    bad = np.zeros(32, np.uint8)
    bad[5] = 0b11000000
    assert oracle.unpack_i2s_block(bad)[0] == ERR_INVALID
    assert oracle.unpack_i2s_block(np.zeros(31, np.uint8))[0] == ERR_SHAPE
    assert oracle.unpack_i2s_block(np.zeros(32, np.uint8), trits_len=127)[0] == ERR_SHAPE


def test_tensor_reads_trailing_scale_and_checks_lengths(oracle):
    """i2s.rs:292-333"""
    payload = np.concatenate([np.full(32, 0b10010101, np.uint8),
                              np.frombuffer(np.float32(1.2188548).tobytes(), np.uint8)])
    rc, t, s = oracle.unpack_i2s_tensor(payload, 128)
    assert rc == 0 and s.view(np.uint32) == np.float32(1.2188548).view(np.uint32)
    assert (t[:32] == 1).all() and (t[32:] == 0).all()
    assert oracle.unpack_i2s_tensor(np.zeros(32, np.uint8), 128)[0] == ERR_SHAPE   # the scale is missing
    assert oracle.unpack_i2s_tensor(np.zeros(100, np.uint8), 100)[0] == ERR_SHAPE  # not a multiple of 128


def test_convert_equals_packing_the_decoded_rows(oracle):
    """convert_i2s_to_tq2_0 (i2s_int8.rs:47-68) against the independent layout statement above and
    the (separately pinned) TQ2_0 row packer; rows that straddle 128-blocks included (k = 192)."""
    rng = np.random.default_rng(21)
    for n, k in ((1, 128), (2, 192), (4, 256), (3, 640), (8, 2560)):
        trits = rng.integers(-1, 2, (n, k)).astype(np.int8)
        payload = i2s_payload(trits, 0.75, pad=28)
        rc, packed, s = oracle.convert_i2s_to_tq2_0(payload, n, k)
        assert rc == 0 and s == np.float32(0.75)
        assert (packed == oracle.pack_matrix(trits, n, k, FMT_TQ2_0)).all()
        assert (oracle.unpack_i2s_tensor(payload, n * k)[1].reshape(n, k) == trits).all()


# ---- the product's host converter ----

def test_product_converter_equals_oracle(oracle):
    rng = np.random.default_rng(22)
    for n, k in ((1, 128), (2, 192), (4, 256), (3, 640), (16, 2560)):
        trits = rng.integers(-1, 2, (n, k)).astype(np.int8)
        payload = i2s_payload(trits, -3.5, pad=28)
        got, s = T.convert_i2s_to_tq2_0(payload, n, k)
        rc, want, s_want = oracle.convert_i2s_to_tq2_0(payload, n, k)
        assert rc == 0 and (got == want).all() and s == s_want
    got, _ = T.convert_i2s_to_tq2_0(np.concatenate([np.frombuffer(REAL_BLOCK, np.uint8), np.zeros(4, np.uint8)]), 1, 128)
    assert T.unpack_rows(got, 1, 128).reshape(-1).tolist() == REAL_TRITS


def test_product_converter_errors():
    ok = i2s_payload(np.zeros(128, np.int8), 1.0)
    with pytest.raises(T.ShapeMismatch) as e:  # the scale is missing
        T.convert_i2s_to_tq2_0(ok[:32], 1, 128)
    assert (e.value.expected, e.value.got) == (36, 32)
    with pytest.raises(T.InvalidInput):        # 100 elements: not a multiple of 128
        T.convert_i2s_to_tq2_0(np.zeros(29, np.uint8), 1, 100)
    bad = ok.copy()
    bad[5] = 0b11000000
    with pytest.raises(T.InvalidInput):        # reserved code
        T.convert_i2s_to_tq2_0(bad, 1, 128)
