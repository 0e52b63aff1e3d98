/*
 * tritium_oracle.h — CPU restatement of the reference's packed-ternary linear path.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the parity checker and the timed CPU
 * baseline. The product (the HIP kernel library and its host adapter) never links,
 * loads or calls it; only the test-suite, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * Every function restates, in plain C, one function of the reference (Rust); the
 * citation beside each declaration is `path:line` under the reference checkout.
 * All floating-point code here must be compiled with -ffp-contract=off and without
 * -ffast-math: the reference's arithmetic is single IEEE-754 binary32 operations in
 * a fixed order and nothing may be fused or re-associated.
 *
 * Parity status: every function below is pinned by a known-answer test, golden bytes
 * or a mathematical invariant in tests/test_oracle_*.py; none is "parity unpinned".
 * What cannot be confirmed without the reference's toolchain is only that the
 * regenerated conformance set is byte-identical to the reference's absent frozen file.
 */
#ifndef TRITIUM_ORACLE_H
#define TRITIUM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* crates/tritium-format/src/lib.rs:144-150 */
#define TO_QK_K 256
#define TO_TQ2_0_BLOCK_BYTES 66
#define TO_TQ1_0_BLOCK_BYTES 54
/* IEEE binary16 1.0: the block scale every host packer on this path writes
 * (crates/tritium-nn/src/layers/linear.rs:166-184, crates/tritium-testkit/src/runner.rs:135-158). */
#define TO_F16_ONE 0x3C00u

/* crates/tritium-core/src/dtype.rs:89-107 — tags used across this build. */
enum { TO_FMT_TQ1_0 = 1, TO_FMT_TQ2_0 = 2 };

/* Return codes. 0 = ok. */
enum {
  TO_OK = 0,
  TO_ERR_SHAPE = 1,       /* a length disagrees with the shape */
  TO_ERR_FORMAT = 2,      /* unsupported format tag */
  TO_ERR_INVALID = 4,     /* input failed validation */
  TO_ERR_BACKEND = 5      /* a packed row decodes outside {-1,0,+1} */
};

/* ---- crates/tritium-format/src/tq2.rs:21-81 ---- */
int to_pack_tq2_0_block(const int8_t *trits256, uint16_t scale_f16, uint8_t *out66);
/* returns TO_ERR_BACKEND when a 2-bit slot holds the reserved code 3 (trit 2). */
int to_unpack_tq2_0_block(const uint8_t *block66, int8_t *trits256, uint16_t *scale_f16);

/* ---- crates/tritium-format/src/tq1.rs:18-30,36-121 ---- */
int to_pack_tq1_0_block(const int8_t *trits256, uint16_t scale_f16, uint8_t *out54);
int to_unpack_tq1_0_block(const uint8_t *block54, int8_t *trits256, uint16_t *scale_f16);

/* ---- crates/tritium-format/src/rows.rs:25-151 ---- */
size_t to_num_blocks(size_t k);
size_t to_row_bytes(size_t k, int format); /* 0 for an unknown format */
int to_pack_row(const int8_t *trits, size_t k, const uint16_t *scales_f16, size_t n_scales,
                int format, uint8_t *out, size_t out_len);
int to_unpack_row(const uint8_t *packed, size_t packed_len, int format, int8_t *trits, size_t k,
                  uint16_t *scales_f16, size_t n_scales);
/* Pack an [n,k] trit matrix row by row with block scale 1.0, as the reference's callers do
 * (crates/tritium-testkit/src/runner.rs:135-158; crates/tritium-nn/src/layers/linear.rs:143-185). */
int to_pack_matrix(const int8_t *trits, size_t n, size_t k, int format, uint8_t *out, size_t out_len);

/* ---- crates/tritium-core/src/reference.rs:25-64 ---- */
int to_reference_mpgemm(const float *act, size_t act_len, const int8_t *trits, size_t w_len,
                        const float *scale_n, size_t scale_len, size_t m, size_t n, size_t k,
                        float *out, size_t out_len);

/* ---- crates/tritium-spec/src/lib.rs:338-378 (== crates/tritium-nn/src/ops/act_quant.rs:94-157) ---- */
void to_quantize_act_int8(const float *act, size_t m, size_t k, float *q_out, float *scale_out);

/* ---- crates/tritium-format/src/i2s.rs:70-101 : unpack_i2s_block (32 bytes -> 128 trits) ---- */
int to_unpack_i2s_block(const uint8_t *block, size_t block_len, int8_t *trits, size_t trits_len);
/* ---- crates/tritium-format/src/i2s.rs:116-158 : unpack_i2s_tensor (quants + trailing f32 scale) ---- */
int to_unpack_i2s_tensor(const uint8_t *payload, size_t payload_len, size_t n_elements, int8_t *trits,
                         size_t trits_len, float *scale);
/* ---- crates/tritium-format/src/i2s_int8.rs:47-68 : convert_i2s_to_tq2_0 ---- */
int to_convert_i2s_to_tq2_0(const uint8_t *payload, size_t payload_len, size_t n, size_t k, uint8_t *out,
                            size_t out_len, float *scale);

/* ---- half::f16::to_f32 (exact) ---- */
float to_f16_to_f32(uint16_t h);
/* ---- crates/tritium-format/src/salt.rs:720-738 : dequant_salt_row over T planes of one row ---- */
int to_salt_dequant_row(const uint8_t *const *planes, size_t t_planes, size_t k, float *out);
/* ---- crates/tritium-nn/src/layers/packed_salt.rs:585-628 : forward over dequantized rows;
 *      planes[p] = plane p of all n rows (crates/tritium-cuda/kernels/tq2_0_add.cu:659-672) ---- */
int to_salt_mpgemm(const uint8_t *const *planes, size_t t_planes, size_t n, size_t k, const float *act,
                   size_t m, float *out);

/* ---- crates/tritium-nn/src/ops/rmsnorm.rs:21-35 : the canonical sum of squares ---- */
float to_sum_squares_canonical(const float *x, size_t n);
/* ---- crates/tritium-nn/src/ops/rmsnorm.rs:43-96 : rmsnorm / rmsnorm_zero_centered ---- */
void to_rmsnorm(const float *x, const float *w, size_t n, float eps, int zero_centered, float *out);
/* ---- crates/tritium-cuda/src/cuda/tests.rs:4692-4725 : host definition of the fused
 *      rmsnorm -> int8 quantization (w is shared by the m rows of x [m,k]) ---- */
void to_rmsnorm_quant(const float *x, const float *w, size_t m, size_t k, float eps, int zero_centered,
                      float *q_out, float *scale_out);

/* ---- crates/tritium-cpu/src/lib.rs:262-300 : upload_weights ----
 * Validates the packed length; for TQ2_0 reports the first row holding a reserved code in
 * *tq2_invalid_row (or -1). The bytes themselves are kept verbatim by the caller. */
int to_cpu_upload_check(const uint8_t *packed, size_t len, size_t n, size_t k, int format,
                        long *tq2_invalid_row);

/* ---- crates/tritium-cpu/src/lib.rs:302-345,181-217 + kernel.rs:49-78,670-678 : mpgemm ----
 * unpack all N*K trits, then the scalar kernel (== reference_mpgemm). The SIMD kernels of the
 * reference are bit-identical to it by the reference's own tests
 * (crates/tritium-cpu/src/kernel.rs:1069-1173), so this is the value oracle for every path. */
int to_cpu_mpgemm(const uint8_t *packed, size_t packed_len, int format, const float *act,
                  size_t act_len, const float *scales, size_t scales_len, size_t m, size_t n,
                  size_t k, float *out, size_t out_len);

/* ---- crates/tritium-spec/src/lib.rs:266-318 : default mpgemm_with_act_quant ----
 * quantize -> mpgemm on int8-valued f32 -> out[m,:] *= act_scale[m]. */
int to_cpu_mpgemm_with_act_quant(const uint8_t *packed, size_t packed_len, int format,
                                 const float *act, size_t act_len, const float *scales,
                                 size_t scales_len, size_t m, size_t n, size_t k, float *out,
                                 size_t out_len);

/* Exact int32 accumulators Σ_k q[m,k]·trit[n,k] for int8 activations (the value the reference's
 * f32 fold holds before its two multiplies: crates/tritium-cpu/src/kernel.rs:588-599,824-828). */
/* mpgemm_projected_vjp, scalar path of the CPU backend (crates/tritium-cpu/src/kernel.rs:82-189):
 * pinned by the reference's known-answer case (crates/tritium-cpu/src/lib.rs:500-533) and against a
 * float64 evaluation of the three sums. grad_bias may be NULL. */
int to_cpu_projected_vjp(const uint8_t *packed, size_t packed_len, int format, const float *act,
                         size_t act_len, const float *scales, size_t scales_len,
                         const float *grad_output, size_t grad_output_len, size_t m, size_t n,
                         size_t k, float *grad_act, size_t grad_act_len, float *grad_w,
                         size_t grad_w_len, float *grad_bias, size_t grad_bias_len);

int to_int8_accumulators(const uint8_t *packed, size_t packed_len, int format, const int8_t *q,
                         size_t m, size_t n, size_t k, int32_t *acc);

/* Additive planes: out = Σ_p mpgemm(plane_p, scales_p) in plane order, f32 adds. The reference has
 * no single function for this at per-channel-scale granularity; it is the composition through
 * TernaryBackend::mpgemm (crates/tritium-spec/src/lib.rs:166-215), one call per plane. */
int to_cpu_mpgemm_planes(const uint8_t *const *packed, const size_t *packed_len, int format,
                         const float *const *scales, size_t planes, const float *act, size_t m,
                         size_t n, size_t k, float *out);
/* int8-activation planes: out[m,n] = (Σ_p ((float)acc_p · s_p[n])) · act_scale[m]; with one plane
 * this is exactly crates/tritium-cpu/src/kernel.rs:921-922 followed by
 * crates/tritium-nn/src/layers/linear.rs:272-277. */
int to_cpu_linear_a8_planes(const uint8_t *const *packed, const size_t *packed_len, int format,
                            const float *const *scales, size_t planes, const float *act, size_t m,
                            size_t n, size_t k, float *out);

/* ---- crates/tritium-testkit/src/vector.rs:113-125 ---- */
int to_accepts_with_floor(float got, float want, float relative, int bit_exact, float floor_);

/* ---- crates/tritium-testkit/src/generate.rs:18-57,65-233 : conformance vectors ---- */
typedef struct to_vector {
  char id[40];
  size_t m, n, k;
  int format;
  float *activation; /* [m*k] */
  int8_t *weights;   /* [n*k] */
  float *scales;     /* [n]   */
  float *expected;   /* [m*n] */
} to_vector;
typedef struct to_vector_set {
  size_t count;
  to_vector *v;
} to_vector_set;
to_vector_set *to_generate_vectors(uint64_t seed, size_t count);
void to_free_vectors(to_vector_set *s);
/* raw generator access for the known-answer tests */
uint64_t to_xorshift64_next(uint64_t *state);

/* bf16 helpers (round-to-nearest-even), used to state bf16-in / bf16-out expectations. */
uint16_t to_f32_to_bf16(float x);
float to_bf16_to_f32(uint16_t h);

/* ---- zero-block bitmaps: crates/tritium-format/src/tq2.rs:101-181 ----
 * One bit per 256-trit block of a packed TQ2_0 row, SET when all 64 code bytes are 0x55 (every trit
 * zero; the scale bytes do not matter); ceil(nb/32) words per row, padding bits never set.
 * to_compute_zero_bitmap: TO_ERR_SHAPE when the row is shorter than nb*66 bytes, or `words` than
 * ceil(nb/32). to_compute_zero_bitmaps: rows `row_bytes` apart; k == 0 -> TO_OK with nothing written;
 * TO_ERR_SHAPE when row_bytes < nb*66, packed_len < n*row_bytes (saturating), or words_len is not
 * n*ceil(nb/32). */
int to_compute_zero_bitmap(const uint8_t *packed_row, size_t row_len, size_t k, uint32_t *words, size_t words_len);
int to_compute_zero_bitmaps(const uint8_t *packed, size_t packed_len, size_t n, size_t k, size_t row_bytes,
                            uint32_t *words, size_t words_len);

/* ---- timed CPU baseline: crates/tritium-cpu/src/kernel.rs:49-78,568-573,577-664,824-1003 ----
 * Same dispatch as the reference: unpack every call; rows chunked at clamp(65536/(n*k),1,m)
 * across `threads` workers; AVX-VNNI/AVX2 int8 kernel when every activation is an integer in
 * [-128,127] and k <= 65536, else the k-order f32 fold. Values equal to_cpu_mpgemm bit for bit.
 * Returns the worker count actually used in *threads_used. */
int to_cpu_mpgemm_fast(const uint8_t *packed, size_t packed_len, int format, const float *act,
                       const float *scales, size_t m, size_t n, size_t k, float *out, int threads,
                       int *threads_used, int *kernel_used);

/* ======================================================================================
 * SALT containers and SALT V2 (salt_oracle.c)
 * ====================================================================================== */
/* FormatError variants of crates/tritium-format/src/lib.rs the SALT readers and writers return, and the
 * SaltV2CodecError / SaltV2CpuError variants of salt_v2.rs and crates/tritium-cpu/src/salt_v2.rs. */
enum {
  TO_SALT_BAD_MAGIC = 20,
  TO_SALT_UNSUPPORTED_VERSION = 21,
  TO_SALT_WRONG_LEN = 22,           /* WrongBlockLen */
  TO_SALT_INVALID_PLANE_TAG = 23,
  TO_SALT_SPARSE_BASE_PLANE = 24,
  TO_SALT_OUT_OF_RANGE = 25,        /* DecodedOutOfRange */
  TO_SALT_NONCANONICAL_INDICES = 26,
  TO_SALT_ROW_TOO_LONG = 27,
  TO_SALT_NONZERO_PADDING = 28,
  TO_SALT_INVALID_DENSITY = 29,
  TO_SALT_TOO_MANY_PLANES = 30,
  TO_SALT_V2_WRONG_PACKED_LENGTH = 40,
  TO_SALT_V2_INVALID_D2_CODE = 41,
  TO_SALT_V2_INVALID_B3_CODE = 42,
  TO_SALT_V2_NONCANONICAL_TRIT_PADDING = 43,
  TO_SALT_V2_S34_NOT_MULTIPLE_OF_FOUR = 44,
  TO_SALT_V2_S34_ZERO_COUNT = 45,
  TO_SALT_V2_NONCANONICAL_BIT_PADDING = 46,
  TO_SALT_V2_NONFINITE_ACTIVATION = 47,
  TO_SALT_V2_NONFINITE_OUTPUT = 48
};
/* crates/tritium-format/src/salt_v2.rs:22-32 (tags as crates/tritium-cuda/kernels/salt_v2.cu:31-52 numbers them) */
enum { TO_SALT_V2_D2 = 0, TO_SALT_V2_B3 = 1, TO_SALT_V2_S34 = 2 };

/* ---- crates/tritium-format/src/sparse.rs ---- */
size_t to_sparse_plane_packed_len(size_t k, size_t nnz);                                             /* :33-34,444-475 */
int to_sparse_from_tq2_0(const uint8_t *packed, size_t packed_len, size_t k, uint16_t *scales, uint32_t *idx,
                         int8_t *sign, size_t *nnz);                                                 /* :235-285 */
int to_sparse_to_tq2_0(size_t k, const uint16_t *scales, size_t n_scales, const uint32_t *idx, const int8_t *sign,
                       size_t nnz, uint8_t *out, size_t out_len);                                    /* :293-340 */
int to_pack_sparse_plane(size_t k, const uint16_t *scales, size_t n_scales, const uint32_t *idx, const int8_t *sign,
                         size_t nnz, uint8_t *out, size_t out_len);                                  /* :444-475 */
int to_unpack_sparse_plane(const uint8_t *bytes, size_t len, size_t *k, uint16_t *scales, size_t scales_cap,
                           uint32_t *idx, int8_t *sign, size_t cap, size_t *nnz);                    /* :92-157,479-481 */
/* ---- crates/tritium-format/src/salt.rs ---- */
int to_pack_salt_row(size_t k, const uint8_t *const *planes, size_t t, uint8_t *out, size_t out_cap, size_t *written); /* :229-241 */
int to_pack_progressive_salt_row(size_t k, const uint8_t *const *planes, size_t t, float max_sparse_density,
                                 uint8_t *out, size_t out_cap, size_t *written);                     /* :253-316 */
int to_packed_salt_row_len(const uint8_t *bytes, size_t len, size_t *row_len);                       /* :352-434,596-598 */
int to_unpack_salt_row_prefix(const uint8_t *bytes, size_t len, size_t max_planes, size_t *k, size_t *planes,
                              uint8_t *dense_out, size_t dense_cap);                                 /* :484-515,669-700 */
/* ---- crates/tritium-format/src/salt_v2.rs ---- */
int to_salt_v2_payload_bytes(int codec, size_t trits, size_t *bytes);                                /* :160-258 */
int to_salt_v2_pack(int codec, const int8_t *trits, size_t n, uint8_t *out, size_t out_len);          /* :268-281,326-349,420-452 */
int to_salt_v2_unpack(int codec, const uint8_t *packed, size_t packed_len, size_t n, int8_t *trits);  /* :289-322,358-392,454-520 */
/* ---- crates/tritium-cpu/src/salt_v2.rs:316-423 (batched as crates/tritium-cuda/kernels/salt_v2.cu:114-216) ---- */
int to_salt_v2_forward(int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                       const uint16_t *scales, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                       size_t n, size_t k, const float *act, size_t m, float *out);
/* ---- crates/tritium-cpu/src/salt_v2.rs:283-300,516-546 ---- */
int to_salt_v2_coefficient(int codec, size_t scale_group, const uint8_t *payload, size_t payload_len,
                           const uint16_t *scales, size_t scale_count, const uint8_t *plane_counts, size_t tiles,
                           size_t n, size_t k, size_t index, float *value);

#ifdef __cplusplus
}
#endif
#endif
