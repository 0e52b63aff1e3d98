// Host-side readers of the SALT weight containers, and the SALT V2 physical codecs.
//
//   * SALT row sidecar "TSLT": a row of T additive TQ2_0 planes with per-256-block f16 scales. Version 1
//     stores the planes dense, back to back; version 2 ("progressive") frames each plane with a tag and a
//     length, and a residual plane may be stored sparse (crates/tritium-format/src/salt.rs:1-19,352-434,484-515).
//   * Sparse residual plane "TSSP": per-block scales plus one u32 per non-zero trit, column in the low 31
//     bits, sign in the top bit, columns strictly ascending (crates/tritium-format/src/sparse.rs:27-41,92-157).
//     A sparse plane expands to exactly the dense TQ2_0 row it was made from (sparse.rs:293-309), which is
//     what the device kernels take: the expansion happens here, once, at load.
//   * SALT V2 codecs: D2 (four linear 2-bit codes per byte), B3 (five little-endian radix-3 digits per
//     byte), S34 (one zero and three signs per group of four, five bits per group)
//     (crates/tritium-format/src/salt_v2.rs:22-32,160-258,268-520).
// Every check the reference's readers make is made here, in their order; all failures are
// TK_ERR_INVALID_INPUT with a message naming the reference's error.
#include <cstring>
#include <vector>

#include "tk_host.h"

namespace {

constexpr size_t kSaltHeader = 10, kSparseHeader = 14, kDescriptor = 5, kBlock = 256, kTq2Block = 66;
constexpr uint32_t kSignBit = 0x80000000u;

inline uint32_t le32(const uint8_t *p) { return (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 | (uint32_t)p[3] << 24; }
inline size_t blocks_of(size_t k) { return (k + kBlock - 1) / kBlock; }

struct RowLayout {
  int version = 0;
  size_t planes = 0, k = 0, plane_bytes = 0, payload_start = 0, encoded_len = 0;
};

// crates/tritium-format/src/salt.rs:352-434
int parse_layout(const uint8_t *b, size_t len, RowLayout *lo) {
  if (len < kSaltHeader) return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: %zu bytes, the header alone is %zu (WrongBlockLen)", len, kSaltHeader);
  if (memcmp(b, "TSLT", 4) != 0) return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: bad magic (SaltBadMagic)");
  lo->version = b[4];
  lo->planes = b[5];
  lo->k = le32(b + 6);
  lo->plane_bytes = blocks_of(lo->k) * kTq2Block;
  if (lo->version == 1) {
    lo->payload_start = kSaltHeader;
    lo->encoded_len = kSaltHeader + lo->planes * lo->plane_bytes;
  } else if (lo->version == 2) {
    lo->payload_start = kSaltHeader + lo->planes * kDescriptor;
    if (lo->payload_start > len)
      return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: descriptors need %zu bytes, got %zu (WrongBlockLen)", lo->payload_start, len);
    size_t payload = 0;
    for (size_t i = 0; i < lo->planes; ++i) {
      const uint8_t *d = b + kSaltHeader + i * kDescriptor;
      if (d[0] == 1 && i == 0) return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: the base plane is tagged sparse (SaltSparseBasePlane)");
      if (d[0] > 1) return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: plane %zu has tag %u (SaltInvalidPlaneTag)", i, (unsigned)d[0]);
      payload += le32(d + 1);
    }
    lo->encoded_len = lo->payload_start + payload;
  } else {
    return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: version %d (UnsupportedSaltVersion)", lo->version);
  }
  if (lo->encoded_len > len)
    return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: encoded length %zu exceeds the %zu bytes given (WrongBlockLen)", lo->encoded_len, len);
  return TK_OK;
}

// crates/tritium-format/src/salt.rs:625-640
int check_dense_plane(const uint8_t *p, size_t len, size_t expected) {
  if (len != expected) return tk_fail(TK_ERR_INVALID_INPUT, "SALT dense plane: %zu bytes, expected %zu (WrongBlockLen)", len, expected);
  for (size_t blk = 0; blk < len; blk += kTq2Block)
    for (size_t i = 0; i < 64; ++i) {
      const uint8_t q = p[blk + i];
      if (q & (q >> 1) & 0x55) return tk_fail(TK_ERR_INVALID_INPUT, "SALT dense plane: reserved 2-bit code (DecodedOutOfRange(2))");
    }
  return TK_OK;
}

// crates/tritium-format/src/sparse.rs:92-157
int parse_sparse(const uint8_t *b, size_t len, size_t *k_out, size_t *nnz_out) {
  if (len < kSparseHeader) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: %zu bytes, the header alone is %zu (WrongBlockLen)", len, kSparseHeader);
  if (memcmp(b, "TSSP", 4) != 0) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: bad magic (SaltBadMagic)");
  if (b[4] != 1) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: version %u (UnsupportedSaltVersion)", (unsigned)b[4]);
  const size_t k = le32(b + 6), nnz = le32(b + 10);
  if (k >= kSignBit) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: k = %zu leaves no room for the sign bit (SaltRowTooLong)", k);
  const size_t entries = kSparseHeader + blocks_of(k) * 2, need = entries + nnz * 4;
  if (len != need) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: %zu bytes, expected %zu (WrongBlockLen)", len, need);
  bool have = false;
  uint32_t prev = 0;
  for (size_t i = 0; i < nnz; ++i) {
    const uint32_t col = le32(b + entries + 4 * i) & ~kSignBit;
    if (col >= k) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: column %u of a row of %zu (DecodedOutOfRange)", col, k);
    if (have && prev >= col) return tk_fail(TK_ERR_INVALID_INPUT, "sparse plane: columns not strictly ascending (SaltNonCanonicalSparseIndices)");
    prev = col;
    have = true;
  }
  *k_out = k;
  *nnz_out = nnz;
  return TK_OK;
}

// A validated sparse plane as the dense TQ2_0 row it stands for (sparse.rs:293-309 through
// crates/tritium-format/src/tq2.rs:21-41): all-zero codes, the listed columns set, each block's scale.
void expand_sparse(const uint8_t *b, size_t k, size_t nnz, uint8_t *row) {
  const size_t nb = blocks_of(k);
  for (size_t blk = 0; blk < nb; ++blk) {
    memset(row + blk * kTq2Block, 0x55, 64);
    row[blk * kTq2Block + 64] = b[kSparseHeader + 2 * blk];
    row[blk * kTq2Block + 65] = b[kSparseHeader + 2 * blk + 1];
  }
  const uint8_t *e = b + kSparseHeader + nb * 2;
  for (size_t i = 0; i < nnz; ++i) {
    const uint32_t enc = le32(e + 4 * i), col = enc & ~kSignBit;
    const size_t blk = col / kBlock, el = col % kBlock;
    // element el of a block: byte (el/128)*32 + el%32, 2-bit slot (el%128)/32
    uint8_t *q = row + blk * kTq2Block + (el / 128) * 32 + el % 32;
    const unsigned shift = 2 * (unsigned)((el % 128) / 32);
    *q = (uint8_t)((*q & ~(3u << shift)) | ((enc & kSignBit ? 0u : 2u) << shift));
  }
}

}  // namespace

extern "C" int tk_salt_row_len(const uint8_t *bytes, size_t len, size_t *row_len) {
  if (!bytes || !row_len) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_row_len: null pointer");
  RowLayout lo;
  if (int rc = parse_layout(bytes, len, &lo)) return rc;
  *row_len = lo.encoded_len;
  return TK_OK;
}

extern "C" int tk_salt_row_info(const uint8_t *bytes, size_t len, size_t *k, size_t *planes, int *version) {
  if (!bytes) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_row_info: null pointer");
  RowLayout lo;
  if (int rc = parse_layout(bytes, len, &lo)) return rc;
  if (k) *k = lo.k;
  if (planes) *planes = lo.planes;
  if (version) *version = lo.version;
  return TK_OK;
}

extern "C" int tk_salt_row_unpack(const uint8_t *bytes, size_t len, size_t max_planes, uint8_t *planes_out,
                                  size_t planes_out_len, size_t *k, size_t *n_planes) {
  if (!bytes || !k || !n_planes) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_row_unpack: null pointer");
  RowLayout lo;
  if (int rc = parse_layout(bytes, len, &lo)) return rc;
  if (len != lo.encoded_len)
    return tk_fail(TK_ERR_INVALID_INPUT, "SALT row: %zu bytes, the row is %zu (WrongBlockLen)", len, lo.encoded_len);
  const size_t keep = lo.planes < max_planes ? lo.planes : max_planes;
  if (keep && (!planes_out || planes_out_len < keep * lo.plane_bytes)) return tk_fail_mismatch(keep * lo.plane_bytes, planes_out_len);
  size_t off = lo.payload_start;
  for (size_t i = 0; i < lo.planes; ++i) {  // every plane is validated, also those beyond max_planes
    const bool framed = lo.version == 2;
    const int tag = framed ? bytes[kSaltHeader + i * kDescriptor] : 0;
    const size_t plen = framed ? le32(bytes + kSaltHeader + i * kDescriptor + 1) : lo.plane_bytes;
    const uint8_t *payload = bytes + off;
    if (tag == 0) {
      if (int rc = check_dense_plane(payload, plen, lo.plane_bytes)) return rc;
      if (i < keep) memcpy(planes_out + i * lo.plane_bytes, payload, lo.plane_bytes);
    } else {
      size_t sk = 0, nnz = 0;
      if (int rc = parse_sparse(payload, plen, &sk, &nnz)) return rc;
      if (sk != lo.k) return tk_fail(TK_ERR_INVALID_INPUT, "SALT row of k = %zu holds a sparse plane of k = %zu (WrongBlockLen)", lo.k, sk);
      if (i < keep) expand_sparse(payload, sk, nnz, planes_out + i * lo.plane_bytes);
    }
    off += plen;
  }
  *k = lo.k;
  *n_planes = keep;
  return TK_OK;
}

extern "C" int tk_sparse_plane_to_tq2_0(const uint8_t *bytes, size_t len, uint8_t *row_out, size_t row_out_len, size_t *k) {
  if (!bytes || !k) return tk_fail(TK_ERR_INVALID_INPUT, "tk_sparse_plane_to_tq2_0: null pointer");
  size_t sk = 0, nnz = 0;
  if (int rc = parse_sparse(bytes, len, &sk, &nnz)) return rc;
  const size_t need = blocks_of(sk) * kTq2Block;
  if (need && (!row_out || row_out_len != need)) return tk_fail_mismatch(need, row_out_len);
  expand_sparse(bytes, sk, nnz, row_out);
  *k = sk;
  return TK_OK;
}

// ------------------------------------------------------------------------------------------
// SALT V2 codecs
// ------------------------------------------------------------------------------------------

extern "C" int tk_salt_v2_payload_bytes(int codec, size_t trits, size_t *bytes) {
  if (!bytes) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_payload_bytes: null pointer");
  switch (codec) {
    case TK_SALT_V2_D2: *bytes = (trits + 3) / 4; return TK_OK;
    case TK_SALT_V2_B3: *bytes = (trits + 4) / 5; return TK_OK;
    case TK_SALT_V2_S34:
      if (trits % 4) return tk_fail(TK_ERR_INVALID_INPUT, "S34 takes whole groups of four trits, got %zu (S34TritCountNotMultipleOfFour)", trits);
      *bytes = (trits / 4 * 5 + 7) / 8;
      return TK_OK;
    default: return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "SALT V2 codec %d", codec);
  }
}

extern "C" int tk_salt_v2_pack(int codec, const int8_t *trits, size_t n, uint8_t *out, size_t out_len) {
  size_t need = 0;
  if (int rc = tk_salt_v2_payload_bytes(codec, n, &need)) return rc;
  if ((!trits && n) || (!out && need)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_pack: null pointer");
  if (out_len != need) return tk_fail_mismatch(need, out_len);
  for (size_t i = 0; i < n; ++i)
    if (trits[i] < -1 || trits[i] > 1) return tk_fail(TK_ERR_INVALID_INPUT, "trit %d at %zu", (int)trits[i], i);
  if (codec == TK_SALT_V2_D2) {
    for (size_t b = 0; b < need; ++b) {
      unsigned q = 0;
      for (size_t s = 0; s < 4; ++s) q |= (b * 4 + s < n ? (unsigned)(trits[b * 4 + s] + 1) : 1u) << (2 * s);
      out[b] = (uint8_t)q;
    }
  } else if (codec == TK_SALT_V2_B3) {
    for (size_t b = 0; b < need; ++b) {
      unsigned v = 0;
      for (size_t s = 5; s-- > 0;) v = v * 3 + (b * 5 + s < n ? (unsigned)(trits[b * 5 + s] + 1) : 1u);  // first trit least significant
      out[b] = (uint8_t)v;
    }
  } else {
    memset(out, 0, need);
    for (size_t gi = 0; gi < n / 4; ++gi) {
      const int8_t *q = trits + gi * 4;
      unsigned zeros = 0, where = 0, sign_bits = 0, signs = 0;
      for (unsigned i = 0; i < 4; ++i) {
        if (q[i] == 0) {
          if (!zeros) where = i;
          ++zeros;
        } else {
          if (q[i] > 0) sign_bits |= 1u << signs;
          ++signs;
        }
      }
      if (zeros != 1) return tk_fail(TK_ERR_INVALID_INPUT, "S34 group %zu holds %u zeros, not one (S34ZeroCount)", gi, zeros);
      const unsigned code = where | (sign_bits << 2);
      const size_t bit = gi * 5;
      const unsigned wide = code << (bit % 8);
      out[bit / 8] |= (uint8_t)wide;
      if (wide >> 8) out[bit / 8 + 1] |= (uint8_t)(wide >> 8);
    }
  }
  return TK_OK;
}

extern "C" int tk_salt_v2_unpack(int codec, const uint8_t *packed, size_t packed_len, size_t n, int8_t *trits) {
  size_t need = 0;
  if (int rc = tk_salt_v2_payload_bytes(codec, n, &need)) return rc;
  if ((!packed && need) || (!trits && n)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_salt_v2_unpack: null pointer");
  if (packed_len != need) return tk_fail(TK_ERR_INVALID_INPUT, "SALT V2 payload: %zu bytes, expected %zu (WrongPackedLength)", packed_len, need);
  if (codec == TK_SALT_V2_D2) {
    for (size_t i = 0; i < need * 4; ++i) {
      const unsigned code = (packed[i / 4] >> (2 * (i % 4))) & 3u;
      if (code == 3) return tk_fail(TK_ERR_INVALID_INPUT, "D2 slot %zu holds the reserved code (InvalidD2Code)", i);
      if (i >= n) {
        if (code != 1) return tk_fail(TK_ERR_INVALID_INPUT, "D2 padding slot %zu is not a zero trit (NonCanonicalTritPadding)", i);
      } else {
        trits[i] = (int8_t)((int)code - 1);
      }
    }
  } else if (codec == TK_SALT_V2_B3) {
    for (size_t b = 0; b < need; ++b) {
      unsigned v = packed[b];
      if (v >= 243) return tk_fail(TK_ERR_INVALID_INPUT, "B3 byte %zu = %u is outside 0..242 (InvalidB3Code)", b, v);
      for (size_t s = 0; s < 5; ++s, v /= 3) {
        const unsigned digit = v % 3;
        if (b * 5 + s >= n) {
          if (digit != 1) return tk_fail(TK_ERR_INVALID_INPUT, "B3 padding digit %zu is not a zero trit (NonCanonicalTritPadding)", b * 5 + s);
        } else {
          trits[b * 5 + s] = (int8_t)((int)digit - 1);
        }
      }
    }
  } else {
    const size_t bits = n / 4 * 5;
    if (bits % 8 && (packed[need - 1] >> (bits % 8)))
      return tk_fail(TK_ERR_INVALID_INPUT, "S34 payload: bits behind the last group are set (NonCanonicalBitPadding)");
    for (size_t gi = 0; gi < n / 4; ++gi) {
      const size_t bit = gi * 5;
      const unsigned word = packed[bit / 8] | (bit / 8 + 1 < need ? (unsigned)packed[bit / 8 + 1] << 8 : 0u);
      const unsigned code = (word >> (bit % 8)) & 31u;
      unsigned signs = code >> 2;
      for (unsigned i = 0; i < 4; ++i) {
        if (i == (code & 3u)) {
          trits[gi * 4 + i] = 0;
        } else {
          trits[gi * 4 + i] = (signs & 1u) ? 1 : -1;
          signs >>= 1;
        }
      }
    }
  }
  return TK_OK;
}
