"""The product's SALT readers and SALT V2 codecs (host code of the library, no GPU) against the oracle's
restatement of crates/tritium-format/src/{salt,sparse,salt_v2}.rs and the reference's known answers."""
import numpy as np
import pytest

import salt_oracle_lib as S
import tritium_amd as T
from test_oracle_salt_formats import lcg_trits, sparse_residual, tq2_row


@pytest.fixture(scope="module")
def so():
    return S.load()


def test_rows_unpack_like_the_oracle_dense_and_sparse(so, oracle):
    for k in (1, 255, 257, 4096):
        planes = [tq2_row(oracle, lcg_trits(k, k), 0x3C00), sparse_residual(oracle, k, 64), sparse_residual(oracle, k, 2),
                  sparse_residual(oracle, k, 33)]
        for packer in (so.pack_salt_row, lambda kk, pp: so.pack_progressive_salt_row(kk, pp, 0.10)):
            rc, data = packer(k, planes)
            assert rc == 0
            assert T.salt_row_len(np.concatenate([data, data])) == data.size
            for mp in (0, 1, 3, 1 << 30):
                kk, got = T.salt_row_unpack(data, mp)
                rc, k2, want = so.unpack_salt_row(data, mp)
                assert rc == 0 and kk == k2 == k and len(got) == len(want) == min(4, mp)
                assert all((g == w).all() for g, w in zip(got, want)) and all((g == p).all() for g, p in zip(got, planes))
    assert bytes(so.pack_salt_row(1, [np.full(66, 0xA5, np.uint8)])[1][:10]) == b"TSLT\x01\x01\x01\0\0\0"
    kk, got = T.salt_row_unpack(np.frombuffer(b"TSLT\x01\x01\x01\0\0\0" + b"\xA5" * 66, np.uint8))
    assert kk == 1 and (got[0] == 0xA5).all()


def test_row_rejections_match_the_oracle(so, oracle):
    k = 4096
    planes = [tq2_row(oracle, lcg_trits(k, 2), 0x3C00), sparse_residual(oracle, k, 64)]
    rc, packed = so.pack_progressive_salt_row(k, planes, 0.10)
    sparse_start = 10 + 2 * 5 + planes[0].size
    cases = {}
    b = packed.copy(); b[10] = 1; cases["SaltSparseBasePlane"] = b
    b = packed.copy(); b[15] = 9; cases["SaltInvalidPlaneTag"] = b
    b = packed.copy(); b[sparse_start + 6: sparse_start + 10] = np.frombuffer(np.uint32(k - 1).tobytes(), np.uint8); cases["WrongBlockLen"] = b
    cases["WrongBlockLen "] = packed[:-1]
    cases["WrongBlockLen  "] = np.concatenate([packed, np.zeros(1, np.uint8)])
    b = packed.copy(); b[0] = ord("X"); cases["SaltBadMagic"] = b
    b = packed.copy(); b[4] = 7; cases["UnsupportedSaltVersion"] = b
    b = packed.copy(); b[20] = 0xFF; cases["DecodedOutOfRange"] = b
    b = packed.copy(); b[sparse_start] = ord("X"); cases["SaltBadMagic "] = b
    first = sparse_start + 14 + 2 * 16
    b = packed.copy(); b[first + 4: first + 8] = b[first: first + 4]; cases["SaltNonCanonicalSparseIndices"] = b
    b = packed.copy(); b[first: first + 4] = np.frombuffer(np.uint32(k).tobytes(), np.uint8); cases["DecodedOutOfRange "] = b
    for name, data in cases.items():
        assert so.unpack_salt_row(data)[0] != 0, name
        with pytest.raises(T.InvalidInput, match=name.strip()):
            T.salt_row_unpack(data)
    with pytest.raises(T.InvalidInput, match="DecodedOutOfRange"):  # omitted planes are validated too
        T.salt_row_unpack(cases["DecodedOutOfRange"], 0)


@pytest.mark.parametrize("k,stride", [(512, 7), (300, 5), (1024, 13), (1, 1), (256, 300)])
def test_sparse_plane_expands_to_the_dense_row(so, oracle, k, stride):
    dense = sparse_residual(oracle, k, stride)
    rc, scales, idx, sign = so.sparse_from_tq2_0(dense, k)
    rc, enc = so.pack_sparse_plane(k, scales, idx, sign)
    kk, row = T.sparse_plane_to_tq2_0(enc)
    assert kk == k and (row == dense).all()
    with pytest.raises(T.InvalidInput, match="WrongBlockLen"):
        T.sparse_plane_to_tq2_0(enc[:-1])


def test_v2_codecs_known_answers_and_oracle_agreement(so):
    assert bytes(T.salt_v2_pack(T.SALT_V2_D2, [-1, 0, 1, -1, 1])) == b"\x24\x56"
    assert bytes(T.salt_v2_pack(T.SALT_V2_B3, [-1, 0, 1, -1, 1, 1])) == b"\xb7\x7a"
    assert bytes(T.salt_v2_pack(T.SALT_V2_S34, [-1, 0, 1, -1, 1, -1, 0, 1])) == b"\xc9\x02"
    rng = np.random.default_rng(0)
    for codec in (T.SALT_V2_D2, T.SALT_V2_B3, T.SALT_V2_S34):
        for n in (0, 4, 8, 12, 100, 256, 1024) + (() if codec == T.SALT_V2_S34 else (1, 5, 6, 173, 255)):
            if codec == T.SALT_V2_S34:
                t = rng.choice([-1, 1], (n // 4, 4)).astype(np.int8)
                t[np.arange(n // 4), rng.integers(0, 4, n // 4)] = 0
                t = t.reshape(-1)
            else:
                t = rng.integers(-1, 2, n).astype(np.int8)
            p = T.salt_v2_pack(codec, t)
            rc, want = so.v2_pack(codec, t)
            assert rc == 0 and p.size == T.salt_v2_payload_bytes(codec, n) and (p == want[:p.size]).all()
            assert (T.salt_v2_unpack(codec, p, n) == t).all()
    u = lambda *b: np.array(b, np.uint8)
    for codec, data, n, err in ((0, u(0b01010111), 1, "InvalidD2Code"), (0, u(0), 1, "NonCanonicalTritPadding"),
                                (0, u(0x55), 5, "WrongPackedLength"), (1, u(243), 5, "InvalidB3Code"),
                                (1, u(0), 1, "NonCanonicalTritPadding"), (1, u(121, 121), 1, "WrongPackedLength"),
                                (2, u(0xC9, 0x82), 8, "NonCanonicalBitPadding"), (2, u(0xC9), 8, "WrongPackedLength"),
                                (2, u(0), 3, "S34TritCountNotMultipleOfFour")):
        assert so.v2_unpack(codec, data, n)[0] != 0
        with pytest.raises(T.InvalidInput, match=err):
            T.salt_v2_unpack(codec, data, n)
    with pytest.raises(T.InvalidInput, match="S34ZeroCount"):
        T.salt_v2_pack(T.SALT_V2_S34, [1, 1, 1, 1])
    with pytest.raises(T.UnsupportedFormat):
        T.salt_v2_payload_bytes(9, 4)
    for code in range(243):
        assert T.salt_v2_pack(1, T.salt_v2_unpack(1, u(code), 5))[0] == code
    for code in range(32):
        assert T.salt_v2_pack(2, T.salt_v2_unpack(2, u(code), 4))[0] == code
