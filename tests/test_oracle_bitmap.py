"""Zero-block bitmaps (crates/tritium-format/src/tq2.rs:101-181): the oracle's restatement against
every case the reference's own tests hold (tq2.rs:187-207, 259-370) and an independent numpy statement;
then the product's host function against the oracle."""
import ctypes as C

import numpy as np
import pytest

import tritium_amd as T
from oracle_lib import FMT_TQ2_0


def _row(oracle, blocks):
    """One packed row from per-block fill values (-1, 0, +1) or explicit 256-trit arrays."""
    trits = np.concatenate([np.full(256, b, np.int8) if np.isscalar(b) else np.asarray(b, np.int8) for b in blocks])
    return oracle.pack_matrix(trits, 1, trits.size, FMT_TQ2_0)


def test_reference_cases(oracle):
    rc, bm = oracle.compute_zero_bitmap(_row(oracle, [0]), 256)          # bitmap_all_zero_block
    assert rc == 0 and bm.tolist() == [1]
    for v in (1, -1):                                                    # bitmap_all_nonzero_block
        rc, bm = oracle.compute_zero_bitmap(_row(oracle, [v]), 256)
        assert rc == 0 and bm.tolist() == [0]
    rc, bm = oracle.compute_zero_bitmap(_row(oracle, [0, 1]), 512)       # bitmap_mixed_blocks
    assert rc == 0 and bm.tolist() == [0b01]
    rc, bm = oracle.compute_zero_bitmap(np.zeros(0, np.uint8), 0)        # bitmap_empty_row
    assert rc == 0 and bm.size == 0
    t = np.zeros(256, np.int8)                                           # bitmap_partial_zero_not_set
    t[128] = 1
    rc, bm = oracle.compute_zero_bitmap(_row(oracle, [t]), 256)
    assert rc == 0 and bm.tolist() == [0]
    packed = np.concatenate([_row(oracle, [0]), _row(oracle, [1])])      # bitmap_multi_row
    rc, bm = oracle.compute_zero_bitmaps(packed, 2, 256, 66)
    assert rc == 0 and bm.tolist() == [1, 0]
    rc, bm = oracle.compute_zero_bitmap(_row(oracle, [0] * 32), 8192)    # bitmap_many_blocks_per_row
    assert rc == 0 and bm.tolist() == [0xFFFFFFFF]
    rc, bm = oracle.compute_zero_bitmap(_row(oracle, [0] * 33), 8448)    # bitmap_spans_multiple_u32_words
    assert rc == 0 and bm.tolist() == [0xFFFFFFFF, 1]


def test_reference_error_cases(oracle):
    """zero_bitmaps_absurd_sizes_are_typed_errors (tq2.rs:187-207): all typed errors, k = 0 is empty."""
    big = (1 << 64) - 1
    assert oracle.compute_zero_bitmaps(np.zeros(0, np.uint8), big, 256, 0, words_len=0)[0] != 0
    assert oracle.compute_zero_bitmaps(np.zeros(0, np.uint8), big, 256, 66, words_len=0)[0] != 0
    assert oracle.compute_zero_bitmaps(np.zeros(1024, np.uint8), 1, 256, 65)[0] != 0
    assert oracle.lib.to_compute_zero_bitmap(None, 0, big, None, 0) != 0
    rc, bm = oracle.compute_zero_bitmaps(np.zeros(0, np.uint8), big, 0, 0, words_len=0)
    assert rc == 0 and bm.size == 0


def test_scale_bytes_and_tail_padding_do_not_matter(oracle):
    """The scale bytes are ignored; a ragged tail (k not a multiple of 256) is zero-padded by the packer,
    so a block whose real trits are all zero is a zero block."""
    row = _row(oracle, [0, 0]).copy()
    row[64:66] = [0x12, 0x34]
    assert oracle.compute_zero_bitmap(row, 512)[1].tolist() == [0b11]
    w = np.zeros((1, 300), np.int8)
    w[0, 10] = -1
    packed = oracle.pack_matrix(w, 1, 300, FMT_TQ2_0)
    assert oracle.compute_zero_bitmap(packed, 300)[1].tolist() == [0b10]


@pytest.mark.parametrize("n,k", [(1, 256), (5, 700), (17, 8448), (3, 256 * 70 - 5)])
def test_against_numpy_statement(oracle, n, k):
    rng = np.random.default_rng(n + k)
    nb = (k + 255) // 256
    zero = rng.random((n, nb)) < 0.4
    w = rng.integers(-1, 2, (n, k)).astype(np.int8)
    for r in range(n):
        for b in range(nb):
            if zero[r, b]:
                w[r, b * 256:(b + 1) * 256] = 0
    is_zero = np.array([[not w[r, b * 256:(b + 1) * 256].any() for b in range(nb)] for r in range(n)])
    packed = oracle.pack_matrix(w, n, k, FMT_TQ2_0)
    rc, bm = oracle.compute_zero_bitmaps(packed, n, k, nb * 66)
    assert rc == 0
    wpr = (nb + 31) // 32
    got = np.array([[(bm[r * wpr + b // 32] >> (b % 32)) & 1 for b in range(nb)] for r in range(n)], bool)
    assert (got == is_zero).all()
    pad = [(bm[r * wpr + (nb - 1) // 32] >> (nb % 32)) if nb % 32 else 0 for r in range(n)]
    assert not any(pad)  # padding bits never set
    # the product's host function: same words, same errors
    mine = T.compute_zero_bitmaps(packed, n, k, nb * 66)
    assert (mine == bm).all()


def test_product_host_function_errors():
    with pytest.raises(T.InvalidInput):
        T.compute_zero_bitmaps(np.zeros(1024, np.uint8), 1, 256, 65)
    with pytest.raises(T.InvalidInput):
        T.compute_zero_bitmaps(np.zeros(0, np.uint8), (1 << 64) - 1, 256, 66)
    assert T.compute_zero_bitmaps(np.zeros(0, np.uint8), 12345, 0, 0).size == 0
