/*
 * tritium_oracle.c — CPU restatement of the reference's packed-ternary linear path.
 *
 * TEST INFRASTRUCTURE ONLY (see tritium_oracle.h). Build with
 *   gcc -O2 -ffp-contract=off -fno-fast-math -fPIC -shared -pthread
 * Each function cites the reference file:line it follows.
 */
#include "tritium_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#if defined(__x86_64__)
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------------- */
/* TQ2_0 block — crates/tritium-format/src/tq2.rs:21-81                        */
/* ------------------------------------------------------------------------- */

/* crates/tritium-format/src/lib.rs:359-371 : LE f16 scale in the last two bytes */
static void write_scale(uint16_t bits, uint8_t *block, size_t len) {
  block[len - 2] = (uint8_t)(bits & 0xFF);
  block[len - 1] = (uint8_t)(bits >> 8);
}
static uint16_t read_scale(const uint8_t *block, size_t len) {
  return (uint16_t)(block[len - 2] | ((uint16_t)block[len - 1] << 8));
}

/* tq2.rs:21-45 : byte c*32+m holds elements c*128+n*32+m (n=0..3) at bits 2n, code = trit+1 */
int to_pack_tq2_0_block(const int8_t *trits, uint16_t scale, uint8_t *out) {
  for (int c = 0; c < 2; ++c) {
    for (int m = 0; m < 32; ++m) {
      uint8_t q = 0;
      for (int n = 0; n < 4; ++n) {
        uint8_t xi = (uint8_t)(trits[c * 128 + n * 32 + m] + 1);
        q |= (uint8_t)((xi & 3) << (2 * n));
      }
      out[c * 32 + m] = q;
    }
  }
  write_scale(scale, out, TO_TQ2_0_BLOCK_BYTES);
  return TO_OK;
}

/* tq2.rs:51-81 ; Trit::from_i8 rejects 2 (crates/tritium-core/src/trit.rs:24-30) */
int to_unpack_tq2_0_block(const uint8_t *block, int8_t *trits, uint16_t *scale) {
  for (int c = 0; c < 2; ++c) {
    for (int l = 0; l < 4; ++l) {
      for (int m = 0; m < 32; ++m) {
        int q = (block[c * 32 + m] >> (2 * l)) & 3;
        int t = q - 1;
        if (t > 1) return TO_ERR_BACKEND;
        trits[c * 128 + l * 32 + m] = (int8_t)t;
      }
    }
  }
  if (scale) *scale = read_scale(block, TO_TQ2_0_BLOCK_BYTES);
  return TO_OK;
}

/* ------------------------------------------------------------------------- */
/* TQ1_0 block — crates/tritium-format/src/tq1.rs:18-30,36-121                 */
/* ------------------------------------------------------------------------- */

static const uint8_t POW3[6] = {1, 3, 9, 27, 81, 243};

/* tq1.rs:20-24 : ceil(acc*256/243) */
static uint8_t tq1_encode(uint16_t acc) { return (uint8_t)(((uint32_t)acc * 256u + 242u) / 243u); }

/* tq1.rs:26-30 : u8 wraparound multiply, then (q*3)>>8, minus one */
static int8_t tq1_decode(uint8_t byte, int n) {
  uint8_t q = (uint8_t)(byte * POW3[n]);
  return (int8_t)((((uint16_t)q * 3u) >> 8) - 1);
}

int to_pack_tq1_0_block(const int8_t *trits, uint16_t scale, uint8_t *out) {
#define XI(i) ((uint16_t)(trits[(i)] + 1))
  for (int m = 0; m < 32; ++m) { /* tq1.rs:53-59 */
    uint16_t acc = 0;
    for (int n = 0; n < 5; ++n) acc = (uint16_t)(acc * 3 + XI(m + n * 32));
    out[m] = tq1_encode(acc);
  }
  for (int m = 0; m < 16; ++m) { /* tq1.rs:61-67 */
    uint16_t acc = 0;
    for (int n = 0; n < 5; ++n) acc = (uint16_t)(acc * 3 + XI(160 + m + n * 16));
    out[32 + m] = tq1_encode(acc);
  }
  for (int j = 0; j < 4; ++j) { /* tq1.rs:69-76 */
    uint16_t acc = 0;
    for (int m = 0; m < 4; ++m) acc = (uint16_t)(acc * 3 + XI(240 + j + m * 4));
    acc = (uint16_t)(acc * 3);
    out[48 + j] = tq1_encode(acc);
  }
#undef XI
  write_scale(scale, out, TO_TQ1_0_BLOCK_BYTES);
  return TO_OK;
}

/* tq1.rs:85-121 */
int to_unpack_tq1_0_block(const uint8_t *block, int8_t *trits, uint16_t *scale) {
  const uint8_t *qs = block;
  const uint8_t *qh = block + 48;
  for (int n = 0; n < 5; ++n)
    for (int m = 0; m < 32; ++m) trits[n * 32 + m] = tq1_decode(qs[m], n);
  for (int n = 0; n < 5; ++n)
    for (int m = 0; m < 16; ++m) trits[160 + n * 16 + m] = tq1_decode(qs[32 + m], n);
  for (int n = 0; n < 4; ++n)
    for (int j = 0; j < 4; ++j) trits[240 + n * 4 + j] = tq1_decode(qh[j], n);
  for (int i = 0; i < 256; ++i)
    if (trits[i] < -1 || trits[i] > 1) return TO_ERR_BACKEND;
  if (scale) *scale = read_scale(block, TO_TQ1_0_BLOCK_BYTES);
  return TO_OK;
}

/* ------------------------------------------------------------------------- */
/* rows — crates/tritium-format/src/rows.rs:25-151                             */
/* ------------------------------------------------------------------------- */

size_t to_num_blocks(size_t k) { return (k + TO_QK_K - 1) / TO_QK_K; } /* rows.rs:25-27 */

static size_t block_bytes(int format) { /* crates/tritium-cpu/src/lib.rs:153-159 */
  if (format == TO_FMT_TQ2_0) return TO_TQ2_0_BLOCK_BYTES;
  if (format == TO_FMT_TQ1_0) return TO_TQ1_0_BLOCK_BYTES;
  return 0;
}

size_t to_row_bytes(size_t k, int format) { return to_num_blocks(k) * block_bytes(format); }

/* rows.rs:61-77 (tq2) / rows.rs:111-127 (tq1): last block zero-padded */
int to_pack_row(const int8_t *trits, size_t k, const uint16_t *scales, size_t n_scales, int format,
                uint8_t *out, size_t out_len) {
  size_t bb = block_bytes(format);
  if (!bb) return TO_ERR_FORMAT;
  size_t nb = to_num_blocks(k);
  if (n_scales != nb) return TO_ERR_SHAPE;   /* rows.rs:37-42 */
  if (out_len != nb * bb) return TO_ERR_SHAPE; /* rows.rs:43-49 */
  int8_t block[TO_QK_K];
  for (size_t i = 0; i < nb; ++i) {
    size_t start = i * TO_QK_K;
    size_t end = start + TO_QK_K < k ? start + TO_QK_K : k;
    size_t cnt = end - start;
    memcpy(block, trits + start, cnt);
    memset(block + cnt, 0, TO_QK_K - cnt);
    if (format == TO_FMT_TQ2_0)
      to_pack_tq2_0_block(block, scales[i], out + i * bb);
    else
      to_pack_tq1_0_block(block, scales[i], out + i * bb);
  }
  return TO_OK;
}

/* rows.rs:87-101 (tq2) / rows.rs:137-151 (tq1): padding discarded */
int to_unpack_row(const uint8_t *packed, size_t packed_len, int format, int8_t *trits, size_t k,
                  uint16_t *scales, size_t n_scales) {
  size_t bb = block_bytes(format);
  if (!bb) return TO_ERR_FORMAT;
  size_t nb = to_num_blocks(k);
  if (n_scales != nb) return TO_ERR_SHAPE;
  if (packed_len != nb * bb) return TO_ERR_SHAPE;
  int8_t block[TO_QK_K];
  for (size_t i = 0; i < nb; ++i) {
    uint16_t s;
    int rc = format == TO_FMT_TQ2_0 ? to_unpack_tq2_0_block(packed + i * bb, block, &s)
                                    : to_unpack_tq1_0_block(packed + i * bb, block, &s);
    if (rc) return rc;
    if (scales) scales[i] = s;
    size_t start = i * TO_QK_K;
    size_t end = start + TO_QK_K < k ? start + TO_QK_K : k;
    memcpy(trits + start, block, end - start);
  }
  return TO_OK;
}

/* crates/tritium-testkit/src/runner.rs:135-158 : per-row pack, unit block scales, rows concatenated */
int to_pack_matrix(const int8_t *trits, size_t n, size_t k, int format, uint8_t *out, size_t out_len) {
  size_t rb = to_row_bytes(k, format);
  if (!block_bytes(format)) return TO_ERR_FORMAT;
  if (out_len != n * rb) return TO_ERR_SHAPE;
  size_t nb = to_num_blocks(k);
  uint16_t *unit = (uint16_t *)malloc((nb ? nb : 1) * sizeof(uint16_t));
  for (size_t i = 0; i < nb; ++i) unit[i] = TO_F16_ONE;
  int rc = TO_OK;
  for (size_t ni = 0; ni < n && !rc; ++ni)
    rc = to_pack_row(trits + ni * k, k, unit, nb, format, out + ni * rb, rb);
  free(unit);
  return rc;
}

/* ------------------------------------------------------------------------- */
/* reference_mpgemm — crates/tritium-core/src/reference.rs:25-64               */
/* ------------------------------------------------------------------------- */

int to_reference_mpgemm(const float *act, size_t act_len, const int8_t *w, size_t w_len,
                        const float *scale_n, size_t scale_len, size_t m, size_t n, size_t k,
                        float *out, size_t out_len) {
  if (act_len != m * k) return TO_ERR_SHAPE; /* reference.rs:32-35, in this order */
  if (w_len != n * k) return TO_ERR_SHAPE;
  if (scale_len != n) return TO_ERR_SHAPE;
  if (out_len != m * n) return TO_ERR_SHAPE;
  for (size_t mi = 0; mi < m; ++mi) {
    const float *arow = act + mi * k;
    for (size_t ni = 0; ni < n; ++ni) {
      const int8_t *wrow = w + ni * k;
      volatile float acc = 0.0f; /* one f32 accumulator, strictly k-order (reference.rs:42-50) */
      for (size_t ki = 0; ki < k; ++ki) {
        if (wrow[ki] == 1)
          acc = acc + arow[ki];
        else if (wrow[ki] == -1)
          acc = acc - arow[ki];
      }
      out[mi * n + ni] = acc * scale_n[ni]; /* reference.rs:51 */
    }
  }
  return TO_OK;
}

/* ------------------------------------------------------------------------- */
/* I2_S — crates/tritium-format/src/i2s.rs, i2s_int8.rs:36-68                  */
/* ------------------------------------------------------------------------- */

/* i2s.rs:70-101 : byte gp supplies positions gp, 32+gp, 64+gp, 96+gp from bit pairs [7:6] .. [1:0];
 * trit = code - 1; code 3 is an error. */
int to_unpack_i2s_block(const uint8_t *block, size_t block_len, int8_t *trits, size_t trits_len) {
  if (block_len != 32) return TO_ERR_SHAPE;   /* WrongBlockLen */
  if (trits_len != 128) return TO_ERR_SHAPE;  /* WrongTritCount */
  for (size_t gp = 0; gp < 32; ++gp)
    for (int group = 0; group < 4; ++group) {
      int shift = 6 - 2 * group;
      unsigned code = (block[gp] >> shift) & 3u;
      if (code == 3u) return TO_ERR_INVALID; /* InvalidI2sCode */
      trits[group * 32 + gp] = (int8_t)((int)code - 1);
    }
  return TO_OK;
}

/* i2s.rs:116-158 : n_elements/4 quant bytes, then one little-endian f32 scale. */
int to_unpack_i2s_tensor(const uint8_t *payload, size_t payload_len, size_t n_elements, int8_t *trits,
                         size_t trits_len, float *scale) {
  if (trits_len != n_elements || n_elements % 128 != 0) return TO_ERR_SHAPE;
  size_t n_quant = n_elements / 4;
  if (payload_len < n_quant + 4) return TO_ERR_SHAPE;
  for (size_t b = 0; b < n_elements / 128; ++b) {
    int rc = to_unpack_i2s_block(payload + b * 32, 32, trits + b * 128, 128);
    if (rc) return rc;
  }
  uint32_t bits = (uint32_t)payload[n_quant] | ((uint32_t)payload[n_quant + 1] << 8) |
                  ((uint32_t)payload[n_quant + 2] << 16) | ((uint32_t)payload[n_quant + 3] << 24);
  memcpy(scale, &bits, 4);
  return TO_OK;
}

/* tq2.rs:101-122 : bit b of word b/32 is set iff every qs byte of block b is 0x55. */
static size_t sat_mul(size_t a, size_t b) {
  size_t r;
  return __builtin_mul_overflow(a, b, &r) ? (size_t)-1 : r;
}

int to_compute_zero_bitmap(const uint8_t *packed_row, size_t row_len, size_t k, uint32_t *words, size_t words_len) {
  const size_t nb = k / TO_QK_K + (k % TO_QK_K != 0);
  const size_t need = sat_mul(nb, TO_TQ2_0_BLOCK_BYTES); /* tq2.rs:105 */
  if (row_len < need) return TO_ERR_SHAPE;               /* FormatError::WrongBlockLen */
  const size_t nwords = nb / 32 + (nb % 32 != 0);
  if (words_len < nwords) return TO_ERR_SHAPE;
  for (size_t w = 0; w < nwords; ++w) words[w] = 0;
  for (size_t b = 0; b < nb; ++b) {
    const uint8_t *qs = packed_row + b * TO_TQ2_0_BLOCK_BYTES;
    int all = 1;
    for (size_t i = 0; i < 64; ++i) all &= qs[i] == 0x55;
    if (all) words[b / 32] |= (uint32_t)1 << (b % 32);
  }
  return TO_OK;
}

/* tq2.rs:134-181 */
int to_compute_zero_bitmaps(const uint8_t *packed, size_t packed_len, size_t n, size_t k, size_t row_bytes,
                            uint32_t *words, size_t words_len) {
  const size_t nb = k / TO_QK_K + (k % TO_QK_K != 0);
  const size_t wpr = nb / 32 + (nb % 32 != 0);
  if (nb == 0) return TO_OK;                                          /* tq2.rs:146-148 */
  if (row_bytes < sat_mul(nb, TO_TQ2_0_BLOCK_BYTES)) return TO_ERR_SHAPE; /* :155-161 */
  if (packed_len < sat_mul(n, row_bytes)) return TO_ERR_SHAPE;           /* :165-171 */
  if (words_len != sat_mul(n, wpr)) return TO_ERR_SHAPE;
  for (size_t r = 0; r < n; ++r) {
    int rc = to_compute_zero_bitmap(packed + r * row_bytes, row_bytes, k, words + r * wpr, wpr);
    if (rc) return rc;
  }
  return TO_OK;
}

/* i2s_int8.rs:47-68 : decode, then pack_tq2_0_row of every row with unit block scales. */
int to_convert_i2s_to_tq2_0(const uint8_t *payload, size_t payload_len, size_t n, size_t k, uint8_t *out,
                            size_t out_len, float *scale) {
  size_t n_elements = n * k;
  int8_t *trits = (int8_t *)malloc(n_elements ? n_elements : 1);
  int rc = to_unpack_i2s_tensor(payload, payload_len, n_elements, trits, n_elements, scale);
  if (!rc) rc = to_pack_matrix(trits, n, k, TO_FMT_TQ2_0, out, out_len);
  free(trits);
  return rc;
}

/* ------------------------------------------------------------------------- */
/* act quant — crates/tritium-spec/src/lib.rs:351-378                          */
/* ------------------------------------------------------------------------- */

/* Rust f32::clamp(min,max): NaN stays NaN. */
static float clampf(float x, float lo, float hi) {
  if (x < lo) return lo;
  if (x > hi) return hi;
  return x;
}

void to_quantize_act_int8(const float *act, size_t m, size_t k, float *q_out, float *scale_out) {
  const float A8_QB = 127.0f; /* lib.rs:341 */
  for (size_t r = 0; r < m; ++r) {
    const float *row = act + r * k;
    float gamma = 0.0f;
    for (size_t c = 0; c < k; ++c) { /* lib.rs:354-360 : `a > gamma`, so NaN never becomes gamma */
      float a = fabsf(row[c]);
      if (a > gamma) gamma = a;
    }
    float *out_row = q_out + r * k;
    if (gamma == 0.0f) { /* lib.rs:362-368 */
      for (size_t c = 0; c < k; ++c) out_row[c] = 0.0f;
      scale_out[r] = 0.0f;
      continue;
    }
    float s = A8_QB / gamma; /* lib.rs:369 : one divide */
    for (size_t c = 0; c < k; ++c) {
      float scaled = row[c] * s;          /* one multiply */
      float rounded = nearbyintf(scaled); /* round_ties_even under the default rounding mode */
      out_row[c] = clampf(rounded, -128.0f, A8_QB);
    }
    scale_out[r] = gamma / A8_QB; /* lib.rs:376 */
  }
}

/* ------------------------------------------------------------------------- */
/* SALT block-scale planes — crates/tritium-format/src/salt.rs:720-738,        */
/* crates/tritium-nn/src/layers/packed_salt.rs:585-628                         */
/* ------------------------------------------------------------------------- */

/* IEEE binary16 -> binary32, exact (half::f16::to_f32). */
float to_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

/* salt.rs:720-738 dequant_salt_row: W[i] = sum over planes, in plane order from 0.0, of
 * f32(block scale) * f32(trit); each plane is one TQ2_0 row of num_blocks(k) blocks. */
int to_salt_dequant_row(const uint8_t *const *planes, size_t t_planes, size_t k, float *out) {
  size_t nb = to_num_blocks(k);
  int8_t *trits = (int8_t *)malloc(k ? k : 1);
  uint16_t *scales = (uint16_t *)malloc((nb ? nb : 1) * sizeof(uint16_t));
  int rc = TO_OK;
  for (size_t i = 0; i < k; ++i) out[i] = 0.0f;
  for (size_t p = 0; p < t_planes && !rc; ++p) {
    rc = to_unpack_row(planes[p], nb * TO_TQ2_0_BLOCK_BYTES, TO_FMT_TQ2_0, trits, k, scales, nb);
    if (rc) break;
    for (size_t i = 0; i < k; ++i) {
      float term = to_f16_to_f32(scales[i / TO_QK_K]) * (float)trits[i];
      out[i] = out[i] + term;
    }
  }
  free(trits);
  free(scales);
  return rc;
}

/* packed_salt.rs:585-628 : out[m,n] = one f32 accumulator over k in order of act[m,k] * W[n,k],
 * W the dequantized row. planes[p] is plane p of all n rows, row-major (the plane-major layout of
 * crates/tritium-cuda/kernels/tq2_0_add.cu:659-672). */
int to_salt_mpgemm(const uint8_t *const *planes, size_t t_planes, size_t n, size_t k, const float *act,
                   size_t m, float *out) {
  size_t rb = to_num_blocks(k) * TO_TQ2_0_BLOCK_BYTES;
  float *w = (float *)malloc((k ? k : 1) * sizeof(float));
  const uint8_t **row = (const uint8_t **)malloc((t_planes ? t_planes : 1) * sizeof(*row));
  int rc = TO_OK;
  for (size_t ni = 0; ni < n && !rc; ++ni) {
    for (size_t p = 0; p < t_planes; ++p) row[p] = planes[p] + ni * rb;
    rc = to_salt_dequant_row(row, t_planes, k, w);
    if (rc) break;
    for (size_t mi = 0; mi < m; ++mi) {
      float acc = 0.0f;
      for (size_t ki = 0; ki < k; ++ki) {
        float prod = act[mi * k + ki] * w[ki];
        acc = acc + prod;
      }
      out[mi * n + ni] = acc;
    }
  }
  free(w);
  free(row);
  return rc;
}

/* ------------------------------------------------------------------------- */
/* RMSNorm — crates/tritium-nn/src/ops/rmsnorm.rs:21-96                        */
/* ------------------------------------------------------------------------- */

/* rmsnorm.rs:21-35 : 256 slots, slot t folds x[t], x[t+256], ... in ascending order (multiply, then
 * add), then a power-of-two tree over the slots (off = 128 .. 1). */
float to_sum_squares_canonical(const float *x, size_t n) {
  float part[256];
  for (int t = 0; t < 256; ++t) part[t] = 0.0f;
  for (size_t i = 0; i < n; ++i) {
    float sq = x[i] * x[i];
    part[i % 256] = part[i % 256] + sq;
  }
  for (int off = 128; off > 0; off >>= 1)
    for (int t = 0; t < off; ++t) part[t] = part[t] + part[t + off];
  return part[0];
}

/* rmsnorm.rs:43-96 : out[i] = x[i] * inv * scale(w[i]) with inv = 1 / sqrt(sum/n + eps);
 * scale(w) = w (rmsnorm) or 1 + w (rmsnorm_zero_centered). n == 0 writes nothing. */
void to_rmsnorm(const float *x, const float *w, size_t n, float eps, int zero_centered, float *out) {
  if (n == 0) return;
  float mean_sq = to_sum_squares_canonical(x, n) / (float)n;
  float inv = 1.0f / sqrtf(mean_sq + eps);
  for (size_t i = 0; i < n; ++i) {
    float sc = zero_centered ? 1.0f + w[i] : w[i];
    float t = x[i] * inv;
    out[i] = t * sc;
  }
}

/* The fused decode step: RMSNorm of each row, then quantize_act_int8 of the result
 * (host definition in crates/tritium-cuda/src/cuda/tests.rs:4692-4725; the launch it replaces:
 * crates/tritium-cuda/src/cuda/mod.rs:1029-1040). */
void to_rmsnorm_quant(const float *x, const float *w, size_t m, size_t k, float eps, int zero_centered,
                      float *q_out, float *scale_out) {
  float *y = (float *)malloc((k ? k : 1) * sizeof(float));
  for (size_t r = 0; r < m; ++r) {
    to_rmsnorm(x + r * k, w, k, eps, zero_centered, y);
    to_quantize_act_int8(y, 1, k, q_out + r * k, scale_out + r);
  }
  free(y);
}

/* ------------------------------------------------------------------------- */
/* CPU backend — crates/tritium-cpu/src/lib.rs:181-217,262-345                 */
/* ------------------------------------------------------------------------- */

int to_cpu_upload_check(const uint8_t *packed, size_t len, size_t n, size_t k, int format,
                        long *tq2_invalid_row) {
  size_t bb = block_bytes(format);
  if (!bb) return TO_ERR_FORMAT;                     /* lib.rs:153-159 */
  size_t row_bytes = to_num_blocks(k) * bb;
  if (len != n * row_bytes) return TO_ERR_INVALID;   /* lib.rs:276-281 */
  long bad = -1;
  if (format == TO_FMT_TQ2_0 && row_bytes != 0) {    /* lib.rs:282-292 */
    for (size_t r = 0; r < n && bad < 0; ++r) {
      const uint8_t *row = packed + r * row_bytes;
      for (size_t b = 0; b < row_bytes / bb && bad < 0; ++b)
        for (int i = 0; i < 64; ++i) {
          uint8_t byte = row[b * bb + i];
          if (byte & (byte >> 1) & 0x55) { bad = (long)r; break; }
        }
    }
  }
  if (tq2_invalid_row) *tq2_invalid_row = bad;
  return TO_OK;
}

/* lib.rs:181-217 : unpack_weights */
static int unpack_weights(const uint8_t *packed, size_t packed_len, int format, size_t n, size_t k,
                          int8_t **out) {
  size_t bb = block_bytes(format);
  if (!bb) return TO_ERR_FORMAT;
  size_t nb = to_num_blocks(k);
  size_t row_bytes = nb * bb;
  if (packed_len != n * row_bytes) return TO_ERR_SHAPE; /* lib.rs:193-198 */
  int8_t *trits = (int8_t *)malloc(n * k ? n * k : 1);
  for (size_t ni = 0; ni < n; ++ni) {
    int rc = to_unpack_row(packed + ni * row_bytes, row_bytes, format, trits + ni * k, k, NULL, nb);
    if (rc) { free(trits); return TO_ERR_BACKEND; } /* lib.rs:213 */
  }
  *out = trits;
  return TO_OK;
}

int to_cpu_mpgemm(const uint8_t *packed, size_t packed_len, int format, const float *act,
                  size_t act_len, const float *scales, size_t scales_len, size_t m, size_t n,
                  size_t k, float *out, size_t out_len) {
  if (act_len != m * k) return TO_ERR_SHAPE;   /* lib.rs:319-324 */
  if (scales_len != n) return TO_ERR_SHAPE;    /* lib.rs:325-330 */
  if (out_len != m * n) return TO_ERR_SHAPE;   /* lib.rs:331-336 */
  int8_t *trits = NULL;
  int rc = unpack_weights(packed, packed_len, format, n, k, &trits); /* lib.rs:339 */
  if (rc) return rc;
  /* kernel.rs:49-78 -> 670-678 : the scalar kernel is reference_mpgemm */
  rc = to_reference_mpgemm(act, act_len, trits, n * k, scales, scales_len, m, n, k, out, out_len);
  free(trits);
  return rc;
}

/* crates/tritium-spec/src/lib.rs:266-318 */
int to_cpu_mpgemm_with_act_quant(const uint8_t *packed, size_t packed_len, int format,
                                 const float *act, size_t act_len, const float *scales,
                                 size_t scales_len, size_t m, size_t n, size_t k, float *out,
                                 size_t out_len) {
  if (act_len != m * k) return TO_ERR_SHAPE;
  if (out_len != m * n) return TO_ERR_SHAPE;
  if (scales_len != n) return TO_ERR_SHAPE;
  float *q = (float *)malloc((m * k ? m * k : 1) * sizeof(float));
  float *as = (float *)malloc((m ? m : 1) * sizeof(float));
  to_quantize_act_int8(act, m, k, q, as);
  int rc = to_cpu_mpgemm(packed, packed_len, format, q, m * k, scales, n, m, n, k, out, out_len);
  if (!rc)
    for (size_t r = 0; r < m; ++r) /* lib.rs:310-315 */
      for (size_t c = 0; c < n; ++c) out[r * n + c] = out[r * n + c] * as[r];
  free(q);
  free(as);
  return rc;
}

/* TernaryBackend::mpgemm_projected_vjp as the CPU backend runs it without SIMD
 * (crates/tritium-cpu/src/lib.rs:347-395 -> crates/tritium-cpu/src/kernel.rs:82-189 and 199-317):
 *   grad_act[m,k]  = sum over n, in order, of  upstream * (trit * scales[n])      (kernel.rs:150-163, 281-293)
 *   grad_w[n,k]    = sum over m, in order, of  upstream * act[m,k]                (kernel.rs:165-177, 295-307)
 *   grad_bias[n]   = sum over m, in order, of  upstream                           (kernel.rs:181-189)
 * with upstream = grad_output[m,n], every product and sum rounded to f32 on its own. Length checks
 * come in the reference's order and nothing is written when one fails; a TQ2_0 plane holding the
 * reserved code is refused before any output is touched (lib.rs:365-370). grad_bias may be NULL. */
int to_cpu_projected_vjp(const uint8_t *packed, size_t packed_len, int format, const float *act,
                         size_t act_len, const float *scales, size_t scales_len,
                         const float *grad_output, size_t grad_output_len, size_t m, size_t n,
                         size_t k, float *grad_act, size_t grad_act_len, float *grad_w,
                         size_t grad_w_len, float *grad_bias, size_t grad_bias_len) {
  int8_t *trits = NULL;
  int rc = unpack_weights(packed, packed_len, format, n, k, &trits);
  if (rc) return rc;
  rc = TO_OK;
  if (act_len != m * k || scales_len != n || grad_output_len != m * n || grad_act_len != m * k ||
      grad_w_len != n * k || (grad_bias && grad_bias_len != n))
    rc = TO_ERR_SHAPE; /* kernel.rs:102-120 */
  if (!rc) {
    for (size_t i = 0; i < m * k; ++i) grad_act[i] = 0.0f; /* kernel.rs:122-123 */
    for (size_t i = 0; i < n * k; ++i) grad_w[i] = 0.0f;
    for (size_t mi = 0; mi < m; ++mi)
      for (size_t ni = 0; ni < n; ++ni) {
        const float upstream = grad_output[mi * n + ni];
        for (size_t ki = 0; ki < k; ++ki) {
          const float projected = (float)trits[ni * k + ki] * scales[ni];
          grad_act[mi * k + ki] = grad_act[mi * k + ki] + upstream * projected;
        }
      }
    for (size_t ni = 0; ni < n; ++ni)
      for (size_t mi = 0; mi < m; ++mi) {
        const float upstream = grad_output[mi * n + ni];
        for (size_t ki = 0; ki < k; ++ki)
          grad_w[ni * k + ki] = grad_w[ni * k + ki] + upstream * act[mi * k + ki];
      }
    if (grad_bias)
      for (size_t ni = 0; ni < n; ++ni) {
        float acc = 0.0f;
        for (size_t mi = 0; mi < m; ++mi) acc = acc + grad_output[mi * n + ni];
        grad_bias[ni] = acc;
      }
  }
  free(trits);
  return rc;
}

int to_int8_accumulators(const uint8_t *packed, size_t packed_len, int format, const int8_t *q,
                         size_t m, size_t n, size_t k, int32_t *acc) {
  int8_t *trits = NULL;
  int rc = unpack_weights(packed, packed_len, format, n, k, &trits);
  if (rc) return rc;
  for (size_t mi = 0; mi < m; ++mi)
    for (size_t ni = 0; ni < n; ++ni) {
      int64_t s = 0;
      for (size_t ki = 0; ki < k; ++ki) s += (int64_t)q[mi * k + ki] * trits[ni * k + ki];
      acc[mi * n + ni] = (int32_t)s;
    }
  free(trits);
  return TO_OK;
}

int to_cpu_mpgemm_planes(const uint8_t *const *packed, const size_t *packed_len, int format,
                         const float *const *scales, size_t planes, const float *act, size_t m,
                         size_t n, size_t k, float *out) {
  float *tmp = (float *)malloc((m * n ? m * n : 1) * sizeof(float));
  for (size_t i = 0; i < m * n; ++i) out[i] = 0.0f;
  int rc = TO_OK;
  for (size_t p = 0; p < planes && !rc; ++p) {
    rc = to_cpu_mpgemm(packed[p], packed_len[p], format, act, m * k, scales[p], n, m, n, k, tmp, m * n);
    if (rc) break;
    if (p == 0)
      memcpy(out, tmp, m * n * sizeof(float));
    else
      for (size_t i = 0; i < m * n; ++i) out[i] = out[i] + tmp[i];
  }
  free(tmp);
  return rc;
}

int to_cpu_linear_a8_planes(const uint8_t *const *packed, const size_t *packed_len, int format,
                            const float *const *scales, size_t planes, const float *act, size_t m,
                            size_t n, size_t k, float *out) {
  float *q = (float *)malloc((m * k ? m * k : 1) * sizeof(float));
  float *as = (float *)malloc((m ? m : 1) * sizeof(float));
  to_quantize_act_int8(act, m, k, q, as);
  int rc = to_cpu_mpgemm_planes(packed, packed_len, format, scales, planes, q, m, n, k, out);
  if (!rc)
    for (size_t r = 0; r < m; ++r)
      for (size_t c = 0; c < n; ++c) out[r * n + c] = out[r * n + c] * as[r];
  free(q);
  free(as);
  return rc;
}

/* ------------------------------------------------------------------------- */
/* tolerance — crates/tritium-testkit/src/vector.rs:113-125                    */
/* ------------------------------------------------------------------------- */

int to_accepts_with_floor(float got, float want, float relative, int bit_exact, float floor_) {
  if (bit_exact) return got == want;
  if (isnan(want) || isnan(got)) return isnan(want) && isnan(got);
  if (isinf(want) || isinf(got)) return got == want;
  float denom = fabsf(want) > floor_ ? fabsf(want) : floor_; /* f32::max */
  return fabsf(got - want) <= relative * denom;
}

/* ------------------------------------------------------------------------- */
/* conformance vectors — crates/tritium-testkit/src/generate.rs                */
/* ------------------------------------------------------------------------- */

uint64_t to_xorshift64_next(uint64_t *state) { /* generate.rs:30-37 */
  uint64_t x = *state;
  x ^= x << 13;
  x ^= x >> 7;
  x ^= x << 17;
  *state = x;
  return x;
}
static uint64_t below(uint64_t *s, uint64_t n) { return to_xorshift64_next(s) % n; } /* :40-42 */
static float gen_activation(uint64_t *s) { return ((float)below(s, 2000) - 1000.0f) / 100.0f; } /* :45-47 */
static float gen_scale(uint64_t *s) { return ((float)below(s, 200) + 1.0f) / 100.0f; }          /* :50-52 */
static int8_t gen_trit(uint64_t *s) { /* :55-57 : from_sign(below(3) as i8 - 1) */
  int v = (int)below(s, 3) - 1;
  return (int8_t)(v > 0 ? 1 : (v < 0 ? -1 : 0));
}

static void build(to_vector *v, const char *id, size_t m, size_t n, size_t k, float *act,
                  int8_t *w, float *sc, int format) { /* generate.rs:65-90 */
  snprintf(v->id, sizeof v->id, "%s", id);
  v->m = m; v->n = n; v->k = k; v->format = format;
  v->activation = act; v->weights = w; v->scales = sc;
  v->expected = (float *)calloc(m * n ? m * n : 1, sizeof(float));
  to_reference_mpgemm(act, m * k, w, n * k, sc, n, m, n, k, v->expected, m * n);
}

static float *dupf(const float *p, size_t n) {
  float *r = (float *)malloc((n ? n : 1) * sizeof(float));
  memcpy(r, p, n * sizeof(float));
  return r;
}
static int8_t *dupi(const int8_t *p, size_t n) {
  int8_t *r = (int8_t *)malloc(n ? n : 1);
  memcpy(r, p, n);
  return r;
}

to_vector_set *to_generate_vectors(uint64_t seed, size_t count) {
  to_vector_set *set = (to_vector_set *)calloc(1, sizeof *set);
  set->count = count + 25;
  set->v = (to_vector *)calloc(set->count, sizeof(to_vector));
  uint64_t rng = seed | 1; /* generate.rs:25-27 */
  char id[40];
  for (size_t i = 0; i < count; ++i) { /* generate.rs:203-229 */
    rng ^= ((uint64_t)i * 0x9E3779B97F4A7C15ull) | 1;
    size_t m = 1 + (size_t)below(&rng, 64);
    size_t n = 1 + (size_t)below(&rng, 32);
    size_t k = 256 * (1 + (size_t)below(&rng, 2));
    int format = (i % 2 == 0) ? TO_FMT_TQ2_0 : TO_FMT_TQ1_0;
    /* generate.rs:93-103 : activation, then weights, then scales */
    float *act = (float *)malloc(m * k * sizeof(float));
    for (size_t j = 0; j < m * k; ++j) act[j] = gen_activation(&rng);
    int8_t *w = (int8_t *)malloc(n * k);
    for (size_t j = 0; j < n * k; ++j) w[j] = gen_trit(&rng);
    float *sc = (float *)malloc(n * sizeof(float));
    for (size_t j = 0; j < n; ++j) sc[j] = gen_scale(&rng);
    snprintf(id, sizeof id, "rand-%zu", i);
    build(&set->v[i], id, m, n, k, act, w, sc, format);
  }
  /* boundary set — generate.rs:108-183 */
  uint64_t brng = 0xB0117DA47ull | 1;
  static const size_t shapes[5][3] = {{1, 1, 256}, {1, 32, 256}, {64, 1, 256}, {64, 32, 512}, {1, 1, 512}};
  size_t o = count;
  for (size_t si = 0; si < 5; ++si) {
    size_t m = shapes[si][0], n = shapes[si][1], k = shapes[si][2];
    float *act = (float *)malloc(m * k * sizeof(float));
    for (size_t j = 0; j < m * k; ++j) act[j] = gen_activation(&brng);
    float *sc = (float *)malloc(n * sizeof(float));
    for (size_t j = 0; j < n; ++j) sc[j] = gen_scale(&brng);
    int8_t *w = (int8_t *)malloc(n * k);
    memset(w, 0, n * k);
    snprintf(id, sizeof id, "boundary-%zu-allzero", si);
    build(&set->v[o++], id, m, n, k, dupf(act, m * k), dupi(w, n * k), dupf(sc, n), TO_FMT_TQ2_0);
    memset(w, 1, n * k);
    snprintf(id, sizeof id, "boundary-%zu-allpos", si);
    build(&set->v[o++], id, m, n, k, dupf(act, m * k), dupi(w, n * k), dupf(sc, n), TO_FMT_TQ2_0);
    memset(w, 0xFF, n * k);
    snprintf(id, sizeof id, "boundary-%zu-allneg", si);
    build(&set->v[o++], id, m, n, k, dupf(act, m * k), dupi(w, n * k), dupf(sc, n), TO_FMT_TQ1_0);
    for (size_t j = 0; j < n * k; ++j) w[j] = gen_trit(&brng);
    snprintf(id, sizeof id, "boundary-%zu-mixed-tq2", si);
    build(&set->v[o++], id, m, n, k, dupf(act, m * k), dupi(w, n * k), dupf(sc, n), TO_FMT_TQ2_0);
    snprintf(id, sizeof id, "boundary-%zu-mixed-tq1", si);
    build(&set->v[o++], id, m, n, k, act, w, sc, TO_FMT_TQ1_0);
  }
  return set;
}

void to_free_vectors(to_vector_set *s) {
  if (!s) return;
  for (size_t i = 0; i < s->count; ++i) {
    free(s->v[i].activation);
    free(s->v[i].weights);
    free(s->v[i].scales);
    free(s->v[i].expected);
  }
  free(s->v);
  free(s);
}

/* ------------------------------------------------------------------------- */
/* bf16 helpers                                                                */
/* ------------------------------------------------------------------------- */

uint16_t to_f32_to_bf16(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7FFFu + lsb;
  return (uint16_t)(u >> 16);
}
float to_bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* ------------------------------------------------------------------------- */
/* timed baseline — crates/tritium-cpu/src/kernel.rs:49-78,568-664,705-1003    */
/* ------------------------------------------------------------------------- */

/* kernel.rs:834-837 */
static int act_is_a8_integer(const float *act, size_t len) {
  for (size_t i = 0; i < len; ++i) {
    float v = act[i];
    if (!(v == truncf(v) && v >= -128.0f && v <= 127.0f)) return 0;
  }
  return 1;
}

/* kernel.rs:568-573 */
static size_t row_chunk(size_t m, size_t n, size_t k) {
  size_t per_row = n * k;
  if (per_row < 1) per_row = 1;
  size_t c = ((size_t)1 << 16) / per_row;
  if (c < 1) c = 1;
  if (c > m) c = m;
  return c;
}

enum { KERN_SCALAR = 0, KERN_AVX2_F32 = 1, KERN_AVX512_F32 = 2, KERN_AVX2_A8 = 3, KERN_VNNI_A8 = 4 };

#if defined(__x86_64__)
/* kernel.rs:705-822 : SIMD decode into a signed buffer, then the k-order f32 fold */
__attribute__((target("avx2"))) static void avx2_f32_rows(const float *act, const int8_t *w,
                                                          const float *scales, size_t m, size_t n,
                                                          size_t k, float *out) {
  size_t k_simd = k - (k % 8);
  float *signed_buf = (float *)malloc((k_simd ? k_simd : 1) * sizeof(float));
  for (size_t mi = 0; mi < m; ++mi) {
    const float *arow = act + mi * k;
    for (size_t ni = 0; ni < n; ++ni) {
      const int8_t *wrow = w + ni * k;
      __m256 zero = _mm256_setzero_ps();
      for (size_t ki = 0; ki < k_simd; ki += 8) {
        __m256 a = _mm256_loadu_ps(arow + ki);
        __m128i lo = _mm_loadl_epi64((const __m128i *)(wrow + ki));
        __m256i t = _mm256_cvtepi8_epi32(lo);
        __m256 posm = _mm256_castsi256_ps(_mm256_cmpeq_epi32(t, _mm256_set1_epi32(1)));
        __m256 negm = _mm256_castsi256_ps(_mm256_cmpeq_epi32(t, _mm256_set1_epi32(-1)));
        __m256 neg_a = _mm256_sub_ps(zero, a);
        __m256 plus = _mm256_blendv_ps(zero, a, posm);
        __m256 sg = _mm256_blendv_ps(plus, neg_a, negm);
        _mm256_storeu_ps(signed_buf + ki, sg);
      }
      volatile float acc = 0.0f;
      for (size_t ki = 0; ki < k_simd; ++ki) acc = acc + signed_buf[ki];
      for (size_t kt = k_simd; kt < k; ++kt) {
        if (wrow[kt] == 1) acc = acc + arow[kt];
        else if (wrow[kt] == -1) acc = acc - arow[kt];
      }
      out[mi * n + ni] = acc * scales[ni];
    }
  }
  free(signed_buf);
}

/* crates/tritium-cpu/src/simd/avx512.rs:73-180 */
__attribute__((target("avx512f,avx512bw,avx512vl"))) static void avx512_f32_rows(
    const float *act, const int8_t *w, const float *scales, size_t m, size_t n, size_t k, float *out) {
  size_t k_simd = k - (k % 16);
  float *signed_buf = (float *)malloc((k_simd ? k_simd : 1) * sizeof(float));
  for (size_t mi = 0; mi < m; ++mi) {
    const float *arow = act + mi * k;
    for (size_t ni = 0; ni < n; ++ni) {
      const int8_t *wrow = w + ni * k;
      for (size_t ki = 0; ki < k_simd; ki += 16) {
        __m512 a = _mm512_loadu_ps(arow + ki);
        __m128i t = _mm_loadu_si128((const __m128i *)(wrow + ki));
        __m128i z = _mm_set1_epi8(0);
        __mmask16 pos = _mm_cmpgt_epi8_mask(t, z);
        __mmask16 neg = _mm_cmpgt_epi8_mask(z, t);
        __m512 plus = _mm512_maskz_mov_ps(pos, a);
        __m512 sg = _mm512_mask_sub_ps(plus, neg, _mm512_setzero_ps(), a);
        _mm512_storeu_ps(signed_buf + ki, sg);
      }
      volatile float acc = 0.0f;
      for (size_t ki = 0; ki < k_simd; ++ki) acc = acc + signed_buf[ki];
      for (size_t kt = k_simd; kt < k; ++kt) {
        if (wrow[kt] == 1) acc = acc + arow[kt];
        else if (wrow[kt] == -1) acc = acc - arow[kt];
      }
      out[mi * n + ni] = acc * scales[ni];
    }
  }
  free(signed_buf);
}

__attribute__((target("avx2"))) static int32_t hsum256(__m256i acc) {
  __m128i lo = _mm256_castsi256_si128(acc);
  __m128i hi = _mm256_extracti128_si256(acc, 1);
  __m128i s = _mm_add_epi32(lo, hi);
  s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x1B));
  s = _mm_add_epi32(s, _mm_shuffle_epi32(s, 0x4E));
  return _mm_cvtsi128_si32(s);
}

/* kernel.rs:856-926 : codes = w+1 in {0,1,2}; Σ(w+1)·a − Σa */
__attribute__((target("avx2"))) static void avx2_a8_rows(const float *act, const int8_t *w,
                                                         const float *scales, size_t m, size_t n,
                                                         size_t k, float *out) {
  size_t k_simd = k - (k % 32);
  int8_t *q8 = (int8_t *)malloc(k ? k : 1);
  __m256i ones16 = _mm256_set1_epi16(1), one8 = _mm256_set1_epi8(1);
  for (size_t mi = 0; mi < m; ++mi) {
    const float *arow = act + mi * k;
    int64_t row_sum = 0;
    for (size_t c = 0; c < k; ++c) { q8[c] = (int8_t)(int32_t)arow[c]; row_sum += q8[c]; }
    for (size_t ni = 0; ni < n; ++ni) {
      const int8_t *wrow = w + ni * k;
      __m256i acc = _mm256_setzero_si256();
      for (size_t ki = 0; ki < k_simd; ki += 32) {
        __m256i wv = _mm256_loadu_si256((const __m256i *)(wrow + ki));
        __m256i av = _mm256_loadu_si256((const __m256i *)(q8 + ki));
        __m256i codes = _mm256_add_epi8(wv, one8);
        __m256i pairs = _mm256_maddubs_epi16(codes, av);
        acc = _mm256_add_epi32(acc, _mm256_madd_epi16(pairs, ones16));
      }
      int64_t total = hsum256(acc);
      for (size_t kt = k_simd; kt < k; ++kt) total += (int64_t)(wrow[kt] + 1) * q8[kt];
      int64_t sg = total - row_sum;
      out[mi * n + ni] = (float)sg * scales[ni]; /* kernel.rs:921-922 */
    }
  }
  free(q8);
}

/* kernel.rs:939-1003 */
__attribute__((target("avx2,avxvnni"))) static void vnni_a8_rows(const float *act, const int8_t *w,
                                                                 const float *scales, size_t m,
                                                                 size_t n, size_t k, float *out) {
  size_t k_simd = k - (k % 32);
  int8_t *q8 = (int8_t *)malloc(k ? k : 1);
  __m256i one8 = _mm256_set1_epi8(1);
  for (size_t mi = 0; mi < m; ++mi) {
    const float *arow = act + mi * k;
    int64_t row_sum = 0;
    for (size_t c = 0; c < k; ++c) { q8[c] = (int8_t)(int32_t)arow[c]; row_sum += q8[c]; }
    for (size_t ni = 0; ni < n; ++ni) {
      const int8_t *wrow = w + ni * k;
      __m256i acc = _mm256_setzero_si256();
      for (size_t ki = 0; ki < k_simd; ki += 32) {
        __m256i wv = _mm256_loadu_si256((const __m256i *)(wrow + ki));
        __m256i av = _mm256_loadu_si256((const __m256i *)(q8 + ki));
        __m256i codes = _mm256_add_epi8(wv, one8);
        acc = _mm256_dpbusd_avx_epi32(acc, codes, av);
      }
      int64_t total = hsum256(acc);
      for (size_t kt = k_simd; kt < k; ++kt) total += (int64_t)(wrow[kt] + 1) * q8[kt];
      int64_t sg = total - row_sum;
      out[mi * n + ni] = (float)sg * scales[ni];
    }
  }
  free(q8);
}
#endif

/* kernel.rs:577-664 : run_chunk's selection order */
static int pick_kernel(const float *act, size_t act_len, size_t k) {
#if defined(__x86_64__)
  __builtin_cpu_init();
  int avx2 = __builtin_cpu_supports("avx2");
  if (avx2 && k <= 65536 && act_is_a8_integer(act, act_len)) {
    if (__builtin_cpu_supports("avxvnni")) return KERN_VNNI_A8;
    return KERN_AVX2_A8;
  }
  if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
      __builtin_cpu_supports("avx512vl"))
    return KERN_AVX512_F32;
  if (avx2) return KERN_AVX2_F32;
#else
  (void)act; (void)act_len; (void)k;
#endif
  return KERN_SCALAR;
}

static void run_chunk(const float *act, const int8_t *w, const float *scales, size_t rows, size_t n,
                      size_t k, float *out, int *kernel_used) {
  int kern = pick_kernel(act, rows * k, k);
  if (kernel_used) *kernel_used = kern;
  switch (kern) {
#if defined(__x86_64__)
    case KERN_VNNI_A8: vnni_a8_rows(act, w, scales, rows, n, k, out); return;
    case KERN_AVX2_A8: avx2_a8_rows(act, w, scales, rows, n, k, out); return;
    case KERN_AVX512_F32: avx512_f32_rows(act, w, scales, rows, n, k, out); return;
    case KERN_AVX2_F32: avx2_f32_rows(act, w, scales, rows, n, k, out); return;
#endif
    default:
      to_reference_mpgemm(act, rows * k, w, n * k, scales, n, rows, n, k, out, rows * n);
  }
}

typedef struct {
  const float *act; const int8_t *w; const float *scales;
  size_t m, n, k, chunk_rows; float *out;
  size_t next; pthread_mutex_t mu; int kernel_used;
} fast_job;

static void *fast_worker(void *p) {
  fast_job *j = (fast_job *)p;
  for (;;) {
    pthread_mutex_lock(&j->mu);
    size_t r0 = j->next;
    j->next += j->chunk_rows;
    pthread_mutex_unlock(&j->mu);
    if (r0 >= j->m) break;
    size_t rows = j->m - r0 < j->chunk_rows ? j->m - r0 : j->chunk_rows;
    int ku;
    run_chunk(j->act + r0 * j->k, j->w, j->scales, rows, j->n, j->k, j->out + r0 * j->n, &ku);
    j->kernel_used = ku;
  }
  return NULL;
}

int to_cpu_mpgemm_fast(const uint8_t *packed, size_t packed_len, int format, const float *act,
                       const float *scales, size_t m, size_t n, size_t k, float *out, int threads,
                       int *threads_used, int *kernel_used) {
  int8_t *trits = NULL;
  int rc = unpack_weights(packed, packed_len, format, n, k, &trits); /* every call, lib.rs:339 */
  if (rc) return rc;
  if (threads_used) *threads_used = 0;
  if (m == 0 || n == 0) { free(trits); return TO_OK; } /* kernel.rs:63-65 */
  fast_job job = {act, trits, scales, m, n, k, row_chunk(m, n, k), out, 0, PTHREAD_MUTEX_INITIALIZER, 0};
  size_t tasks = (m + job.chunk_rows - 1) / job.chunk_rows;
  int nt = threads < 1 ? 1 : threads;
  if ((size_t)nt > tasks) nt = (int)tasks;
  if (nt > 256) nt = 256;
  if (nt == 1) {
    fast_worker(&job);
  } else {
    pthread_t th[256];
    for (int i = 0; i < nt; ++i) pthread_create(&th[i], NULL, fast_worker, &job);
    for (int i = 0; i < nt; ++i) pthread_join(th[i], NULL);
  }
  if (threads_used) *threads_used = nt;
  if (kernel_used) *kernel_used = job.kernel_used;
  free(trits);
  return TO_OK;
}
