// Host-side TQ2_0 / TQ1_0 row packers: the caller-side half of the path (what TernaryLinear does
// before upload_weights, crates/tritium-nn/src/layers/linear.rs:143-185). Written against the
// format definition (crates/tritium-format/src/tq2.rs:15-18, tq1.rs:1-9), block scale f16 1.0.
#include <cstring>
#include <vector>

#include "tk_host.h"

namespace {

constexpr size_t kBlock = 256;
constexpr uint8_t kF16OneLo = 0x00, kF16OneHi = 0x3C;

inline size_t block_bytes(int format) {
  return format == TK_FORMAT_TQ2_0 ? 66 : (format == TK_FORMAT_TQ1_0 ? 54 : 0);
}

// 2-bit code per trit, four strided elements per byte.
void pack_block_tq2(const int8_t *t, uint8_t *out) {
  for (size_t byte = 0; byte < 64; ++byte) {
    const size_t half = byte / 32, col = byte % 32;
    unsigned q = 0;
    for (unsigned slot = 0; slot < 4; ++slot) q |= (unsigned)(t[half * 128 + slot * 32 + col] + 1) << (2 * slot);
    out[byte] = (uint8_t)q;
  }
  out[64] = kF16OneLo;
  out[65] = kF16OneHi;
}

// Base-3 fixed point: a byte stores ceil(v * 256 / 243) for a 5-digit ternary number v (most
// significant digit first); the last four bytes hold 4 digits each, shifted up one digit.
inline uint8_t tq1_byte(unsigned v) { return (uint8_t)((v * 256u + 242u) / 243u); }

void pack_block_tq1(const int8_t *t, uint8_t *out) {
  for (size_t col = 0; col < 32; ++col) {
    unsigned v = 0;
    for (size_t d = 0; d < 5; ++d) v = v * 3 + (unsigned)(t[d * 32 + col] + 1);
    out[col] = tq1_byte(v);
  }
  for (size_t col = 0; col < 16; ++col) {
    unsigned v = 0;
    for (size_t d = 0; d < 5; ++d) v = v * 3 + (unsigned)(t[160 + d * 16 + col] + 1);
    out[32 + col] = tq1_byte(v);
  }
  for (size_t col = 0; col < 4; ++col) {
    unsigned v = 0;
    for (size_t d = 0; d < 4; ++d) v = v * 3 + (unsigned)(t[240 + d * 4 + col] + 1);
    out[48 + col] = tq1_byte(v * 3);
  }
  out[52] = kF16OneLo;
  out[53] = kF16OneHi;
}

inline int tq1_digit(uint8_t byte, unsigned d) {
  static const unsigned pow3[5] = {1, 3, 9, 27, 81};
  const unsigned q = (byte * pow3[d]) & 0xFFu;
  return (int)((q * 3u) >> 8) - 1;
}

bool unpack_block(const uint8_t *blk, int format, int8_t *t) {
  if (format == TK_FORMAT_TQ2_0) {
    for (size_t byte = 0; byte < 64; ++byte) {
      const size_t half = byte / 32, col = byte % 32;
      for (unsigned slot = 0; slot < 4; ++slot) {
        const int code = (blk[byte] >> (2 * slot)) & 3;
        if (code == 3) return false;
        t[half * 128 + slot * 32 + col] = (int8_t)(code - 1);
      }
    }
    return true;
  }
  for (size_t e = 0; e < 160; ++e) t[e] = (int8_t)tq1_digit(blk[e % 32], (unsigned)(e / 32));
  for (size_t e = 0; e < 80; ++e) t[160 + e] = (int8_t)tq1_digit(blk[32 + e % 16], (unsigned)(e / 16));
  for (size_t e = 0; e < 16; ++e) t[240 + e] = (int8_t)tq1_digit(blk[48 + e % 4], (unsigned)(e / 4));
  return true;
}

}  // namespace

extern "C" size_t tk_packed_len(size_t n, size_t k, int format) {
  // 0 for an unsupported format and for a shape whose byte count does not fit size_t
  size_t row, total;
  if (k > (size_t)-1 - kBlock) return 0;
  if (__builtin_mul_overflow((k + kBlock - 1) / kBlock, block_bytes(format), &row)) return 0;
  if (__builtin_mul_overflow(n, row, &total)) return 0;
  return total;
}

// compute_zero_bitmaps (crates/tritium-format/src/tq2.rs:134-181): one bit per 256-trit block and row,
// set when the block's 64 code bytes are all 0x55. Word `r * ceil(nb/32) + b/32`, bit `b % 32`.
extern "C" int tk_compute_zero_bitmaps(const uint8_t *packed, size_t packed_len, size_t n, size_t k, size_t row_bytes,
                                       uint32_t *words, size_t words_len) {
  const size_t nb = k / kBlock + (k % kBlock != 0), wpr = nb / 32 + (nb % 32 != 0);
  if (nb == 0) return TK_OK;  // nothing to describe, whatever n says (tq2.rs:146-148)
  size_t min_row, need, want;
  if (__builtin_mul_overflow(nb, (size_t)66, &min_row) || row_bytes < min_row)
    return tk_fail(TK_ERR_INVALID_INPUT, "zero bitmap: row of %zu bytes is shorter than the %zu blocks of k=%zu", row_bytes, nb, k);
  if (__builtin_mul_overflow(n, row_bytes, &need) || packed_len < need)
    return tk_fail(TK_ERR_INVALID_INPUT, "zero bitmap: %zu bytes do not hold %zu rows of %zu", packed_len, n, row_bytes);
  if (__builtin_mul_overflow(n, wpr, &want) || words_len != want) return tk_fail_mismatch(want, words_len);
  if ((!packed && need) || (!words && want)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_compute_zero_bitmaps: null pointer");
  std::memset(words, 0, want * sizeof(uint32_t));
  for (size_t r = 0; r < n; ++r)
    for (size_t b = 0; b < nb; ++b) {
      const uint8_t *qs = packed + r * row_bytes + b * 66;
      bool zero = true;
      for (size_t i = 0; i < 64 && zero; ++i) zero = qs[i] == 0x55;
      if (zero) words[r * wpr + b / 32] |= 1u << (b % 32);
    }
  return TK_OK;
}

extern "C" int tk_pack_rows(const int8_t *trits, size_t trits_len, size_t n, size_t k, int format, uint8_t *out,
                            size_t out_len) {
  const size_t bb = block_bytes(format);
  if (!bb) return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "tk_pack_rows: unsupported format %d", format);
  if ((!trits && trits_len) || (!out && out_len)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_pack_rows: null pointer");
  if (trits_len != n * k) return tk_fail_mismatch(n * k, trits_len);
  const size_t nb = (k + kBlock - 1) / kBlock;
  if (out_len != n * nb * bb) return tk_fail_mismatch(n * nb * bb, out_len);
  int8_t block[kBlock];
  for (size_t row = 0; row < n; ++row) {
    for (size_t b = 0; b < nb; ++b) {
      const size_t start = b * kBlock;
      const size_t cnt = k - start < kBlock ? k - start : kBlock;
      for (size_t e = 0; e < cnt; ++e) {
        const int8_t v = trits[row * k + start + e];
        if (v < -1 || v > 1) return tk_fail(TK_ERR_INVALID_INPUT, "tk_pack_rows: weight %d outside {-1,0,1}", (int)v);
        block[e] = v;
      }
      std::memset(block + cnt, 0, kBlock - cnt);  // the tail of the last block is zero-padded
      uint8_t *dst = out + (row * nb + b) * bb;
      if (format == TK_FORMAT_TQ2_0) pack_block_tq2(block, dst); else pack_block_tq1(block, dst);
    }
  }
  return TK_OK;
}

extern "C" int tk_unpack_rows(const uint8_t *packed, size_t packed_len, size_t n, size_t k, int format, int8_t *trits,
                              size_t trits_len) {
  const size_t bb = block_bytes(format);
  if (!bb) return tk_fail(TK_ERR_UNSUPPORTED_FORMAT, "tk_unpack_rows: unsupported format %d", format);
  if ((!packed && packed_len) || (!trits && trits_len)) return tk_fail(TK_ERR_INVALID_INPUT, "tk_unpack_rows: null pointer");
  const size_t nb = (k + kBlock - 1) / kBlock;
  if (packed_len != n * nb * bb) return tk_fail_mismatch(n * nb * bb, packed_len);
  if (trits_len != n * k) return tk_fail_mismatch(n * k, trits_len);
  int8_t block[kBlock];
  for (size_t row = 0; row < n; ++row)
    for (size_t b = 0; b < nb; ++b) {
      if (!unpack_block(packed + (row * nb + b) * bb, format, block))
        return tk_fail(TK_ERR_BACKEND, "unpack row %zu: decoded value 2 outside ternary range", row);
      const size_t start = b * kBlock;
      const size_t cnt = k - start < kBlock ? k - start : kBlock;
      std::memcpy(trits + row * k + start, block, cnt);
    }
  return TK_OK;
}

// ------------------------------------------------------------------------------------------
// I2_S (the BitNet GGUF tensor type 36) -> TQ2_0 rows, once at load:
// convert_i2s_to_tq2_0 (crates/tritium-format/src/i2s_int8.rs:36-68) over unpack_i2s_tensor
// (crates/tritium-format/src/i2s.rs:70-158). The payload is n*k/4 quant bytes followed by one
// little-endian f32 per-tensor scale; the quants are 32-byte blocks of 128 elements in the flat
// [n,k] row-major order, byte gp of a block holding the elements gp, 32+gp, 64+gp, 96+gp of the
// block in its bit pairs [7:6], [5:4], [3:2], [1:0]; code = trit + 1, code 3 is reserved.
// ------------------------------------------------------------------------------------------

extern "C" size_t tk_i2s_payload_len(size_t n, size_t k) {
  size_t elems;
  if (__builtin_mul_overflow(n, k, &elems) || elems % 128 != 0) return 0;
  return elems / 4 + 4;
}

extern "C" int tk_convert_i2s_to_tq2_0(const uint8_t *payload, size_t payload_len, size_t n, size_t k, uint8_t *out,
                                       size_t out_len, float *scale) {
  size_t elems;
  if (__builtin_mul_overflow(n, k, &elems)) return tk_fail(TK_ERR_INVALID_INPUT, "I2_S element count overflows");
  if (elems % 128 != 0)  // i2s.rs:122-127
    return tk_fail(TK_ERR_INVALID_INPUT, "I2_S tensor of %zu elements is not a multiple of 128", elems);
  const size_t quant_bytes = elems / 4, need = quant_bytes + 4;
  if (payload_len < need) return tk_fail_mismatch(need, payload_len);  // i2s.rs:128-135
  const size_t nb = (k + kBlock - 1) / kBlock, want_out = n * nb * 66;
  if (out_len != want_out) return tk_fail_mismatch(want_out, out_len);
  if ((!payload && payload_len) || (!out && out_len) || !scale)
    return tk_fail(TK_ERR_INVALID_INPUT, "tk_convert_i2s_to_tq2_0: null pointer");
  int8_t block[kBlock];
  for (size_t row = 0; row < n; ++row)
    for (size_t b = 0; b < nb; ++b) {
      const size_t start = b * kBlock;
      const size_t cnt = k - start < kBlock ? k - start : kBlock;
      for (size_t e = 0; e < cnt; ++e) {
        const size_t flat = row * k + start + e;          // position in the flat row-major tensor
        const size_t within = flat & 127, gp = within & 31, group = within >> 5;
        const unsigned code = (payload[(flat >> 7) * 32 + gp] >> (6 - 2 * group)) & 3u;
        if (code == 3u) return tk_fail(TK_ERR_INVALID_INPUT, "I2_S code 0b11 at element %zu", flat);
        block[e] = (int8_t)((int)code - 1);
      }
      std::memset(block + cnt, 0, kBlock - cnt);
      pack_block_tq2(block, out + (row * nb + b) * 66);
    }
  uint32_t bits = (uint32_t)payload[quant_bytes] | ((uint32_t)payload[quant_bytes + 1] << 8) |
                  ((uint32_t)payload[quant_bytes + 2] << 16) | ((uint32_t)payload[quant_bytes + 3] << 24);
  std::memcpy(scale, &bits, 4);
  return TK_OK;
}
