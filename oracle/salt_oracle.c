/*
 * salt_oracle.c — CPU restatement of the reference's SALT containers and SALT V2 arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY (see tritium_oracle.h): the parity checker for the product's readers and
 * kernels, and the writer the tests use to make inputs. Never linked into or called by the product.
 *
 * Part 1: the sparse residual plane (crates/tritium-format/src/sparse.rs) and the SALT row sidecar,
 *         legacy v1 and progressive v2 (crates/tritium-format/src/salt.rs).
 * Part 2: the SALT V2 physical codecs D2 / B3 / S34 (crates/tritium-format/src/salt_v2.rs:268-520) and
 *         the exact scalar matrix-vector product and coefficient reconstruction over allocation tiles
 *         (crates/tritium-cpu/src/salt_v2.rs:283-423, crates/tritium-cuda/kernels/salt_v2.cu:114-216).
 *
 * Parity status: pinned by the reference's own known answers (tests/test_oracle_salt.py): the v1 row
 * bytes "TSLT\x01\x01\x01\0\0\0"+0xA5.. (salt.rs tests), the codec bytes [0x24,0x56], [0xb7,0x7a],
 * [0xc9,0x02] and every rejection case of salt_v2.rs's tests, the cancellation-before-scale answer and
 * the non-finite rejections of crates/tritium-cpu/src/salt_v2.rs's tests, exhaustive round trips of all
 * 243 B3 and 32 S34 codes, and an independent dense float64 product. No function here is unpinned.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "tritium_oracle.h"

/* ===================================================================================== */
/* Part 1: sparse plane + SALT row sidecar                                                */
/* ===================================================================================== */

#define SPARSE_HEADER 14u /* sparse.rs:33-34 : magic(4) version(1) pad(1) k u32 nnz u32 */
#define SALT_HEADER 10u   /* salt.rs:44-45  : magic(4) version(1) planes(1) k u32 */
#define SIGN_BIT 0x80000000u

static uint32_t rd32(const uint8_t *p) { return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24); }
static void wr32(uint8_t *p, uint32_t v) {
  p[0] = (uint8_t)v;
  p[1] = (uint8_t)(v >> 8);
  p[2] = (uint8_t)(v >> 16);
  p[3] = (uint8_t)(v >> 24);
}

size_t to_sparse_plane_packed_len(size_t k, size_t nnz) { return SPARSE_HEADER + to_num_blocks(k) * 2 + nnz * 4; }

/* sparse.rs:263-285 validate_zero_padding */
static int zero_padding_ok(const uint8_t *packed, size_t k) {
  size_t used = k % TO_QK_K;
  if (!used) return 1;
  int8_t trits[TO_QK_K];
  uint16_t sc;
  if (to_unpack_tq2_0_block(packed + (to_num_blocks(k) - 1) * TO_TQ2_0_BLOCK_BYTES, trits, &sc)) return 0;
  for (size_t i = used; i < TO_QK_K; ++i)
    if (trits[i] != 0) return 0;
  return 1;
}

/* sparse.rs:235-261 sparse_from_tq2_0. idx / sign need room for k entries. */
int to_sparse_from_tq2_0(const uint8_t *packed, size_t packed_len, size_t k, uint16_t *scales, uint32_t *idx,
                         int8_t *sign, size_t *nnz) {
  if (k >= SIGN_BIT) return TO_SALT_ROW_TOO_LONG;
  size_t nb = to_num_blocks(k);
  int8_t *trits = (int8_t *)malloc(k ? k : 1);
  int rc = to_unpack_row(packed, packed_len, TO_FMT_TQ2_0, trits, k, scales, nb);
  if (rc) {
    free(trits);
    return rc == TO_ERR_BACKEND ? TO_SALT_OUT_OF_RANGE : TO_SALT_WRONG_LEN;
  }
  if (!zero_padding_ok(packed, k)) {
    free(trits);
    return TO_SALT_NONZERO_PADDING;
  }
  size_t c = 0;
  for (size_t i = 0; i < k; ++i)
    if (trits[i] != 0) {
      idx[c] = (uint32_t)i;
      sign[c] = trits[i];
      ++c;
    }
  *nnz = c;
  free(trits);
  return TO_OK;
}

/* sparse.rs:311-340 validate_sparse_plane */
static int validate_sparse(size_t k, size_t n_scales, const uint32_t *idx, const int8_t *sign, size_t nnz) {
  if (k >= SIGN_BIT) return TO_SALT_ROW_TOO_LONG;
  if (n_scales != to_num_blocks(k)) return TO_SALT_WRONG_LEN;
  for (size_t i = 1; i < nnz; ++i)
    if (idx[i - 1] >= idx[i]) return TO_SALT_NONCANONICAL_INDICES;
  for (size_t i = 0; i < nnz; ++i) {
    if (idx[i] >= k) return TO_SALT_OUT_OF_RANGE;
    if (sign[i] != 1 && sign[i] != -1) return TO_SALT_OUT_OF_RANGE;
  }
  return TO_OK;
}

/* sparse.rs:293-309 sparse_to_tq2_0 */
int to_sparse_to_tq2_0(size_t k, const uint16_t *scales, size_t n_scales, const uint32_t *idx, const int8_t *sign,
                       size_t nnz, uint8_t *out, size_t out_len) {
  int rc = validate_sparse(k, n_scales, idx, sign, nnz);
  if (rc) return rc;
  int8_t *trits = (int8_t *)calloc(k ? k : 1, 1);
  for (size_t i = 0; i < nnz; ++i) trits[idx[i]] = sign[i];
  rc = to_pack_row(trits, k, scales, n_scales, TO_FMT_TQ2_0, out, out_len);
  free(trits);
  return rc ? TO_SALT_WRONG_LEN : TO_OK;
}

/* sparse.rs:444-475 pack_sparse_plane */
int to_pack_sparse_plane(size_t k, const uint16_t *scales, size_t n_scales, const uint32_t *idx, const int8_t *sign,
                         size_t nnz, uint8_t *out, size_t out_len) {
  int rc = validate_sparse(k, n_scales, idx, sign, nnz);
  if (rc) return rc;
  if (out_len != to_sparse_plane_packed_len(k, nnz)) return TO_SALT_WRONG_LEN;
  memcpy(out, "TSSP", 4);
  out[4] = 1;
  out[5] = 0;
  wr32(out + 6, (uint32_t)k);
  wr32(out + 10, (uint32_t)nnz);
  uint8_t *p = out + SPARSE_HEADER;
  for (size_t b = 0; b < n_scales; ++b, p += 2) {
    p[0] = (uint8_t)scales[b];
    p[1] = (uint8_t)(scales[b] >> 8);
  }
  for (size_t i = 0; i < nnz; ++i, p += 4) wr32(p, sign[i] == 1 ? idx[i] : (idx[i] | SIGN_BIT));
  return TO_OK;
}

/* sparse.rs:92-157 SparsePlaneRef::parse: every check, in the reference's order */
static int sparse_parse(const uint8_t *bytes, size_t len, size_t *k_out, size_t *nnz_out) {
  if (len < SPARSE_HEADER) return TO_SALT_WRONG_LEN;
  if (memcmp(bytes, "TSSP", 4) != 0) return TO_SALT_BAD_MAGIC;
  if (bytes[4] != 1) return TO_SALT_UNSUPPORTED_VERSION;
  size_t k = rd32(bytes + 6);
  if (k >= SIGN_BIT) return TO_SALT_ROW_TOO_LONG;
  size_t nnz = rd32(bytes + 10);
  size_t required = SPARSE_HEADER + to_num_blocks(k) * 2 + nnz * 4;
  if (len != required) return TO_SALT_WRONG_LEN;
  const uint8_t *e = bytes + SPARSE_HEADER + to_num_blocks(k) * 2;
  int have_prev = 0;
  uint32_t prev = 0;
  for (size_t i = 0; i < nnz; ++i) {
    uint32_t col = rd32(e + 4 * i) & ~SIGN_BIT;
    if (col >= k) return TO_SALT_OUT_OF_RANGE;
    if (have_prev && prev >= col) return TO_SALT_NONCANONICAL_INDICES;
    prev = col;
    have_prev = 1;
  }
  *k_out = k;
  *nnz_out = nnz;
  return TO_OK;
}

/* sparse.rs:479-481 unpack_sparse_plane (parse + to_owned). scales room: num_blocks(k); idx/sign: nnz. */
int to_unpack_sparse_plane(const uint8_t *bytes, size_t len, size_t *k, uint16_t *scales, size_t scales_cap,
                           uint32_t *idx, int8_t *sign, size_t cap, size_t *nnz) {
  int rc = sparse_parse(bytes, len, k, nnz);
  if (rc) return rc;
  size_t nb = to_num_blocks(*k);
  if (nb > scales_cap || *nnz > cap) return TO_ERR_SHAPE;
  for (size_t b = 0; b < nb; ++b) scales[b] = (uint16_t)(bytes[SPARSE_HEADER + 2 * b] | (bytes[SPARSE_HEADER + 2 * b + 1] << 8));
  const uint8_t *e = bytes + SPARSE_HEADER + nb * 2;
  for (size_t i = 0; i < *nnz; ++i) {
    uint32_t enc = rd32(e + 4 * i);
    idx[i] = enc & ~SIGN_BIT;
    sign[i] = (enc & SIGN_BIT) ? -1 : 1;
  }
  return TO_OK;
}

/* salt.rs:625-640 validate_dense_plane */
static int validate_dense_plane(const uint8_t *payload, size_t len, size_t expected) {
  if (len != expected) return TO_SALT_WRONG_LEN;
  for (size_t b = 0; b + TO_TQ2_0_BLOCK_BYTES <= len; b += TO_TQ2_0_BLOCK_BYTES)
    for (size_t i = 0; i < TO_QK_K / 4; ++i)
      for (int sh = 0; sh < 8; sh += 2)
        if (((payload[b + i] >> sh) & 3) == 3) return TO_SALT_OUT_OF_RANGE;
  return TO_OK;
}

/* salt.rs:229-241 pack_salt_row (legacy v1): t dense planes back to back. *written = bytes produced. */
int to_pack_salt_row(size_t k, const uint8_t *const *planes, size_t t, uint8_t *out, size_t out_cap, size_t *written) {
  if (t > 255) return TO_SALT_TOO_MANY_PLANES;
  if (k > 0xFFFFFFFFu) return TO_SALT_ROW_TOO_LONG;
  size_t pb = to_num_blocks(k) * TO_TQ2_0_BLOCK_BYTES;
  for (size_t p = 0; p < t; ++p) {
    int rc = validate_dense_plane(planes[p], pb, pb);
    if (rc) return rc;
  }
  size_t need = SALT_HEADER + t * pb;
  if (out_cap < need) return TO_ERR_SHAPE;
  memcpy(out, "TSLT", 4);
  out[4] = 1;
  out[5] = (uint8_t)t;
  wr32(out + 6, (uint32_t)k);
  for (size_t p = 0; p < t; ++p) memcpy(out + SALT_HEADER + p * pb, planes[p], pb);
  *written = need;
  return TO_OK;
}

/* salt.rs:253-316 pack_progressive_salt_row (v2): plane 0 dense; a residual goes sparse when its density
 * is strictly below max_sparse_density (sparse.rs:404-420) AND its encoded bytes are fewer than dense. */
int to_pack_progressive_salt_row(size_t k, const uint8_t *const *planes, size_t t, float max_sparse_density,
                                 uint8_t *out, size_t out_cap, size_t *written) {
  if (!isfinite(max_sparse_density) || max_sparse_density < 0.0f || max_sparse_density > 1.0f) return TO_SALT_INVALID_DENSITY;
  if (t > 255) return TO_SALT_TOO_MANY_PLANES;
  if (k > 0xFFFFFFFFu) return TO_SALT_ROW_TOO_LONG;
  size_t nb = to_num_blocks(k), pb = nb * TO_TQ2_0_BLOCK_BYTES;
  for (size_t p = 0; p < t; ++p) {
    int rc = validate_dense_plane(planes[p], pb, pb);
    if (rc) return rc;
  }
  uint8_t *tags = (uint8_t *)calloc(t ? t : 1, 1);
  uint8_t **enc = (uint8_t **)calloc(t ? t : 1, sizeof(*enc));
  size_t *lens = (size_t *)calloc(t ? t : 1, sizeof(*lens));
  uint16_t *scales = (uint16_t *)malloc((nb ? nb : 1) * 2);
  uint32_t *idx = (uint32_t *)malloc((k ? k : 1) * 4);
  int8_t *sign = (int8_t *)malloc(k ? k : 1);
  int rc = TO_OK;
  for (size_t p = 0; p < t && !rc; ++p) {
    lens[p] = pb;
    if (p == 0) continue;
    size_t nnz = 0;
    int r = to_sparse_from_tq2_0(planes[p], pb, k, scales, idx, sign, &nnz);
    if (r == TO_SALT_NONZERO_PADDING) continue; /* stays dense */
    if (r) {
      rc = r;
      break;
    }
    float density = k == 0 ? 0.0f : (float)nnz / (float)k;
    if (!(density < max_sparse_density)) continue;
    size_t sl = to_sparse_plane_packed_len(k, nnz);
    if (sl >= pb) continue;
    enc[p] = (uint8_t *)malloc(sl);
    rc = to_pack_sparse_plane(k, scales, nb, idx, sign, nnz, enc[p], sl);
    tags[p] = 1;
    lens[p] = sl;
  }
  if (!rc) {
    size_t need = SALT_HEADER + t * 5;
    for (size_t p = 0; p < t; ++p) need += lens[p];
    if (out_cap < need) rc = TO_ERR_SHAPE;
    else {
      memcpy(out, "TSLT", 4);
      out[4] = 2;
      out[5] = (uint8_t)t;
      wr32(out + 6, (uint32_t)k);
      uint8_t *d = out + SALT_HEADER;
      for (size_t p = 0; p < t; ++p, d += 5) {
        d[0] = tags[p];
        wr32(d + 1, (uint32_t)lens[p]);
      }
      for (size_t p = 0; p < t; ++p) {
        memcpy(d, tags[p] ? enc[p] : planes[p], lens[p]);
        d += lens[p];
      }
      *written = need;
    }
  }
  for (size_t p = 0; p < t; ++p) free(enc[p]);
  free(tags);
  free(enc);
  free(lens);
  free(scales);
  free(idx);
  free(sign);
  return rc;
}

/* salt.rs:352-434 parse_salt_row_layout */
typedef struct {
  int version;
  size_t planes, k, plane_bytes, payload_start, encoded_len;
} SaltLayout;

static int salt_layout(const uint8_t *bytes, size_t len, SaltLayout *lo) {
  if (len < SALT_HEADER) return TO_SALT_WRONG_LEN;
  if (memcmp(bytes, "TSLT", 4) != 0) return TO_SALT_BAD_MAGIC;
  lo->version = bytes[4];
  lo->planes = bytes[5];
  lo->k = rd32(bytes + 6);
  lo->plane_bytes = to_num_blocks(lo->k) * TO_TQ2_0_BLOCK_BYTES;
  if (lo->version == 1) {
    lo->payload_start = SALT_HEADER;
    lo->encoded_len = SALT_HEADER + lo->planes * lo->plane_bytes;
  } else if (lo->version == 2) {
    lo->payload_start = SALT_HEADER + lo->planes * 5;
    if (lo->payload_start > len) return TO_SALT_WRONG_LEN;
    size_t payload = 0;
    for (size_t i = 0; i < lo->planes; ++i) {
      const uint8_t *d = bytes + SALT_HEADER + i * 5;
      if (d[0] == 1 && i == 0) return TO_SALT_SPARSE_BASE_PLANE;
      if (d[0] > 1) return TO_SALT_INVALID_PLANE_TAG;
      payload += rd32(d + 1);
    }
    lo->encoded_len = lo->payload_start + payload;
  } else {
    return TO_SALT_UNSUPPORTED_VERSION;
  }
  if (lo->encoded_len > len) return TO_SALT_WRONG_LEN;
  return TO_OK;
}

/* salt.rs:596-598 packed_salt_row_len */
int to_packed_salt_row_len(const uint8_t *bytes, size_t len, size_t *row_len) {
  SaltLayout lo;
  int rc = salt_layout(bytes, len, &lo);
  if (rc) return rc;
  *row_len = lo.encoded_len;
  return TO_OK;
}

/* salt.rs:484-515 PackedSaltRowRef::parse + salt.rs:669-700 unpack_salt_row_prefix: every plane is validated,
 * the first min(planes, max_planes) are written as dense TQ2_0 rows, back to back, into dense_out. */
int to_unpack_salt_row_prefix(const uint8_t *bytes, size_t len, size_t max_planes, size_t *k, size_t *planes,
                              uint8_t *dense_out, size_t dense_cap) {
  SaltLayout lo;
  int rc = salt_layout(bytes, len, &lo);
  if (rc) return rc;
  if (len != lo.encoded_len) return TO_SALT_WRONG_LEN;
  size_t keep = lo.planes < max_planes ? lo.planes : max_planes;
  size_t off = lo.payload_start;
  size_t nb = to_num_blocks(lo.k);
  uint16_t *scales = (uint16_t *)malloc((nb ? nb : 1) * 2);
  for (size_t i = 0; i < lo.planes && !rc; ++i) {
    int tag = 0;
    size_t plen = lo.plane_bytes;
    if (lo.version == 2) {
      tag = bytes[SALT_HEADER + i * 5];
      plen = rd32(bytes + SALT_HEADER + i * 5 + 1);
    }
    const uint8_t *payload = bytes + off;
    if (tag == 0) {
      rc = validate_dense_plane(payload, plen, lo.plane_bytes);
      if (!rc && i < keep) {
        if ((i + 1) * lo.plane_bytes > dense_cap) rc = TO_ERR_SHAPE;
        else memcpy(dense_out + i * lo.plane_bytes, payload, lo.plane_bytes);
      }
    } else {
      size_t sk = 0, nnz = 0;
      rc = sparse_parse(payload, plen, &sk, &nnz);
      if (!rc && sk != lo.k) rc = TO_SALT_WRONG_LEN;
      if (!rc && i < keep) {
        if ((i + 1) * lo.plane_bytes > dense_cap) rc = TO_ERR_SHAPE;
        else {
          uint32_t *idx = (uint32_t *)malloc((nnz ? nnz : 1) * 4);
          int8_t *sign = (int8_t *)malloc(nnz ? nnz : 1);
          size_t k2, n2;
          rc = to_unpack_sparse_plane(payload, plen, &k2, scales, nb, idx, sign, nnz, &n2);
          if (!rc) rc = to_sparse_to_tq2_0(lo.k, scales, nb, idx, sign, nnz, dense_out + i * lo.plane_bytes, lo.plane_bytes);
          free(idx);
          free(sign);
        }
      }
    }
    off += plen;
  }
  free(scales);
  if (rc) return rc;
  *k = lo.k;
  *planes = keep;
  return TO_OK;
}

/* ===================================================================================== */
/* Part 2: SALT V2                                                                        */
/* ===================================================================================== */

/* salt_v2.rs:160-258 SaltV2Codec::ledger : physical bytes of a payload of `trits` logical trits */
int to_salt_v2_payload_bytes(int codec, size_t trits, size_t *bytes) {
  if (codec == TO_SALT_V2_D2) *bytes = (trits + 3) / 4;
  else if (codec == TO_SALT_V2_B3) *bytes = (trits + 4) / 5;
  else if (codec == TO_SALT_V2_S34) {
    if (trits % 4) return TO_SALT_V2_S34_NOT_MULTIPLE_OF_FOUR;
    *bytes = (trits / 4 * 5 + 7) / 8;
  } else return TO_ERR_FORMAT;
  return TO_OK;
}

/* salt_v2.rs:268-281 pack_d2, :326-349 pack_b3, :420-452 pack_s34 (+ write_s34_code :483-493) */
int to_salt_v2_pack(int codec, const int8_t *trits, size_t n, uint8_t *out, size_t out_len) {
  size_t need;
  int rc = to_salt_v2_payload_bytes(codec, n, &need);
  if (rc) return rc;
  if (out_len != need) return TO_SALT_V2_WRONG_PACKED_LENGTH;
  if (codec == TO_SALT_V2_D2) {
    memset(out, 0x55, need);
    for (size_t i = 0; i < n; ++i) {
      int sh = 2 * (int)(i % 4);
      out[i / 4] = (uint8_t)((out[i / 4] & ~(3u << sh)) | ((unsigned)(trits[i] + 1) << sh));
    }
  } else if (codec == TO_SALT_V2_B3) {
    for (size_t b = 0; b < need; ++b) {
      unsigned code = 0, place = 1;
      for (size_t s = 0; s < 5; ++s) {
        size_t ti = b * 5 + s;
        unsigned digit = ti < n ? (unsigned)(trits[ti] + 1) : 1u;
        code += digit * place;
        place *= 3;
      }
      out[b] = (uint8_t)code;
    }
  } else {
    memset(out, 0, need);
    for (size_t gi = 0; gi < n / 4; ++gi) {
      const int8_t *gp = trits + gi * 4;
      int zeros = 0, zi = 0;
      for (int i = 0; i < 4; ++i)
        if (gp[i] == 0) {
          if (!zeros) zi = i;
          ++zeros;
        }
      if (zeros != 1) return TO_SALT_V2_S34_ZERO_COUNT;
      unsigned code = (unsigned)zi, si = 0;
      for (int i = 0; i < 4; ++i) {
        if (gp[i] == 0) continue;
        if (gp[i] == 1) code |= 1u << (2 + si);
        ++si;
      }
      size_t bit = gi * 5, byte = bit / 8, sh = bit % 8;
      unsigned shifted = code << sh;
      out[byte] |= (uint8_t)shifted;
      if (sh + 5 > 8) out[byte + 1] |= (uint8_t)(shifted >> 8);
    }
  }
  return TO_OK;
}

/* salt_v2.rs:289-322 unpack_d2_into, :358-392 unpack_b3_into, :454-481 unpack_s34_into: canonical decode */
int to_salt_v2_unpack(int codec, const uint8_t *packed, size_t packed_len, size_t n, int8_t *trits) {
  size_t need;
  int rc = to_salt_v2_payload_bytes(codec, n, &need);
  if (rc) return rc;
  if (packed_len != need) return TO_SALT_V2_WRONG_PACKED_LENGTH;
  if (codec == TO_SALT_V2_D2) {
    for (size_t i = 0; i < need * 4; ++i) {
      unsigned code = (packed[i / 4] >> (2 * (i % 4))) & 3u;
      if (code == 3) return TO_SALT_V2_INVALID_D2_CODE;
      if (i >= n) {
        if (code != 1) return TO_SALT_V2_NONCANONICAL_TRIT_PADDING;
        continue;
      }
      trits[i] = (int8_t)((int)code - 1);
    }
  } else if (codec == TO_SALT_V2_B3) {
    for (size_t b = 0; b < need; ++b) {
      if (packed[b] >= 243) return TO_SALT_V2_INVALID_B3_CODE;
      unsigned code = packed[b];
      for (size_t s = 0; s < 5; ++s) {
        unsigned digit = code % 3;
        code /= 3;
        size_t ti = b * 5 + s;
        if (ti >= n) {
          if (digit != 1) return TO_SALT_V2_NONCANONICAL_TRIT_PADDING;
          continue;
        }
        trits[ti] = (int8_t)((int)digit - 1);
      }
    }
  } else {
    size_t bits = n / 4 * 5, pad = (8 - bits % 8) % 8;
    if (pad && (packed[need - 1] & (uint8_t)(0xFFu << (8 - pad)))) return TO_SALT_V2_NONCANONICAL_BIT_PADDING;
    for (size_t gi = 0; gi < n / 4; ++gi) {
      size_t bit = gi * 5, byte = bit / 8, sh = bit % 8;
      unsigned word = packed[byte] | (byte + 1 < need ? (unsigned)packed[byte + 1] << 8 : 0u);
      unsigned code = (word >> sh) & 31u, zi = code & 3u, si = 0;
      for (unsigned i = 0; i < 4; ++i) {
        if (i == zi) {
          trits[gi * 4 + i] = 0;
          continue;
        }
        trits[gi * 4 + i] = (code & (1u << (2 + si))) ? 1 : -1;
        ++si;
      }
    }
  }
  return TO_OK;
}

/* The tensor as the reference's runtimes hold it (salt_v2.cu:114-131): `payload` = the codec bytes of
 * every plane, tile after tile, planes of a tile in order; `scales` = one f16 per (plane, scale group),
 * same order; plane_counts[tile] in 1..3. Tiles cover the row-major coefficients of the [n,k] matrix,
 * 256 at a time (the last may be shorter). Offsets: a tile whose planes start at running plane index
 * `begin` has its plane j at payload offset begin*bytes(256) + j*bytes(len) and its scales at
 * begin*groups(256) + j*groups(len) (salt_v2.cu:175-190). */
typedef struct {
  size_t begin, len, planes;
} TileRef;

static int tile_ref(const uint8_t *plane_counts, size_t tiles, size_t total, size_t tile, TileRef *t) {
  if (tile >= tiles) return TO_ERR_SHAPE;
  size_t begin = 0;
  for (size_t i = 0; i < tile; ++i) begin += plane_counts[i];
  t->begin = begin;
  t->planes = plane_counts[tile];
  t->len = total - tile * 256 < 256 ? total - tile * 256 : 256;
  return TO_OK;
}

static int decode_plane(int codec, const uint8_t *payload, size_t payload_len, const TileRef *t, size_t j, int8_t *trits) {
  size_t full, cur;
  int rc = to_salt_v2_payload_bytes(codec, 256, &full);
  if (!rc) rc = to_salt_v2_payload_bytes(codec, t->len, &cur);
  if (rc) return rc;
  size_t base = t->begin * full + j * cur;
  if (base + cur > payload_len) return TO_ERR_SHAPE;
  return to_salt_v2_unpack(codec, payload + base, cur, t->len, trits);
}

/* crates/tritium-cpu/src/salt_v2.rs:316-423 salt_v2_matvec_into, for m activation rows (the CUDA kernel's
 * batch, salt_v2.cu:133-214): per output row, segments (tile x scale group x row) in ascending coefficient
 * order; per segment, planes ascending; per plane, one f32 accumulator over the columns (add / subtract /
 * skip), ONE multiply by the f16 scale, one add into the output accumulator. A non-finite activation, or any
 * accumulator that leaves the finite range, rejects the call before/without storing (salt_v2.rs:952-1012). */
int to_salt_v2_forward(int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                       const uint16_t *scales, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                       size_t n, size_t k, const float *act, size_t m, float *out) {
  if (scale_group == 0) return TO_ERR_SHAPE;
  const size_t total = n * k;
  if (tiles != (total + 255) / 256) return TO_ERR_SHAPE;
  for (size_t i = 0; i < m * k; ++i)
    if (!isfinite(act[i])) return TO_SALT_V2_NONFINITE_ACTIVATION;
  const size_t full_groups = (256 + scale_group - 1) / scale_group;
  int8_t trits[3][256];
  float *res = (float *)malloc((m * n ? m * n : 1) * sizeof(float));
  int rc = TO_OK;
  for (size_t mi = 0; mi < m && !rc; ++mi) {
    const float *a = act + mi * k;
    size_t loaded_tile = (size_t)-1;
    TileRef t = {0, 0, 0};
    for (size_t row = 0; row < n && !rc; ++row) {
      const size_t row_base = row * k, row_end = row_base + k;
      float accumulator = 0.0f;
      size_t c = row_base;
      while (c < row_end && !rc) {
        const size_t tile = c / 256, local = c - tile * 256;
        if (tile != loaded_tile) {
          rc = tile_ref(plane_counts, tiles, total, tile, &t);
          for (size_t j = 0; j < t.planes && !rc; ++j) rc = decode_plane(codec, payload, payload_len, &t, j, trits[j]);
          if (rc) break;
          loaded_tile = tile;
        }
        const size_t group = local / scale_group;
        size_t group_end = (group + 1) * scale_group;
        if (group_end > t.len) group_end = t.len;
        size_t seg = group_end - local;
        if (seg > row_end - c) seg = row_end - c;
        const size_t cur_groups = (t.len + scale_group - 1) / scale_group;
        for (size_t j = 0; j < t.planes; ++j) {
          const size_t si = t.begin * full_groups + j * cur_groups + group;
          if (si >= scale_count) {
            rc = TO_ERR_SHAPE;
            break;
          }
          float group_acc = 0.0f;
          for (size_t o = 0; o < seg; ++o) {
            const int tr = trits[j][local + o];
            if (tr < 0) group_acc = group_acc - a[c - row_base + o];
            else if (tr > 0) group_acc = group_acc + a[c - row_base + o];
            if (!isfinite(group_acc)) rc = TO_SALT_V2_NONFINITE_OUTPUT;
          }
          const float contribution = group_acc * to_f16_to_f32(scales[si]);
          if (!isfinite(contribution)) rc = TO_SALT_V2_NONFINITE_OUTPUT;
          accumulator = accumulator + contribution;
          if (!isfinite(accumulator)) rc = TO_SALT_V2_NONFINITE_OUTPUT;
          if (rc) break;
        }
        c += seg;
      }
      res[mi * n + row] = accumulator;
    }
  }
  if (!rc) memcpy(out, res, m * n * sizeof(float));
  free(res);
  return rc;
}

/* crates/tritium-cpu/src/salt_v2.rs:283-300 salt_v2_coefficient / salt_v2.cu:218-304 gather: the f32 sum over
 * the tile's planes, ascending, of (trit as f32) * f16 scale -- i.e. add or subtract the scale. */
int to_salt_v2_coefficient(int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                           const uint16_t *scales, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                           size_t n, size_t k, size_t index, float *value) {
  const size_t total = n * k;
  if (index >= total) return TO_SALT_OUT_OF_RANGE;
  if (scale_group == 0 || tiles != (total + 255) / 256) return TO_ERR_SHAPE;
  TileRef t;
  int8_t trits[256];
  int rc = tile_ref(plane_counts, tiles, total, index / 256, &t);
  if (rc) return rc;
  const size_t local = index % 256, group = local / scale_group;
  const size_t full_groups = (256 + scale_group - 1) / scale_group, cur_groups = (t.len + scale_group - 1) / scale_group;
  float acc = 0.0f;
  for (size_t j = 0; j < t.planes; ++j) {
    rc = decode_plane(codec, payload, payload_len, &t, j, trits);
    if (rc) return rc;
    const size_t si = t.begin * full_groups + j * cur_groups + group;
    if (si >= scale_count) return TO_ERR_SHAPE;
    const float s = to_f16_to_f32(scales[si]);
    if (trits[local] < 0) acc = acc - s;
    else if (trits[local] > 0) acc = acc + s;
  }
  *value = acc;
  return TO_OK;
}
